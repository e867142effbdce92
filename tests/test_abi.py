"""The C-ABI library loads without a GPU, exports what include/gptq_hip.h declares, and its
host-side logic (dispatcher, argument checks) behaves.  No kernel is launched here."""
import ctypes
import os
import re

import pytest

from autogptq.tvm_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "gptq_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gptq_hip_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.lib()
    names = declared_functions()
    assert set(names) == set(_lib.ABI_SYMBOLS)
    for name in names:
        assert getattr(lib, name) is not None
    assert lib.gptq_hip_abi_version() == _lib.ABI_VERSION


def test_plan_struct_matches_header():
    text = open(os.path.join(ROOT, "include", "gptq_hip.h")).read()
    body = re.search(r"typedef struct gptq_hip_plan \{(.*?)\} gptq_hip_plan;", text, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        typ, names = decl.rsplit(" ", 1)[0], decl.split(" ", 1)[1]
        typ = "size_t" if decl.startswith("size_t") else "int"
        for nm in names.replace("int", "").replace("size_t", "").split(","):
            fields.append((nm.strip(), typ))
    assert [f for f, _ in fields] == [f for f, _ in _lib.Plan._fields_]
    for (_, typ), (_, ct) in zip(fields, _lib.Plan._fields_):
        assert ct is (ctypes.c_size_t if typ == "size_t" else ctypes.c_int)


def test_strerror_texts():
    assert _lib.strerror(0) == "ok"
    for code in (-1, -2, -3, -4):
        assert _lib.strerror(code) not in ("ok", "unknown status")
    assert _lib.strerror(-99) == "unknown status"


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("M", [1, 2, 3, 5, 8, 16, 17, 64, 128, 256, 1000])
@pytest.mark.parametrize("KN", [(4096, 4096), (4096, 11008), (11008, 4096), (9216, 36864), (36864, 9216), (64, 32)])
@pytest.mark.parametrize("gs", [128, -1])
def test_select_plans_are_consistent(bits, M, KN, gs):
    K, N = KN
    if gs != -1 and K % gs != 0:
        gs = 32
    for act in (False, True):
        p = _lib.select(M, K, N, bits, gs, act)
        assert p.kernel in (_lib.KERNEL_GROUPED, _lib.KERNEL_STREAM)
        if p.kernel == _lib.KERNEL_GROUPED:
            # one or two rows, or up to eight packed into one or two operand tiles (contiguous groups only)
            assert M <= 8 and 1 <= p.row_tiles <= 8 and p.m_blocks == 1
            if M > 2:
                assert not act or gs == -1
                assert p.row_tiles == (4 if M <= 4 else 8) and p.split_k <= 3 and p.block >= 16 * p.row_tiles
        else:
            assert p.row_tiles in (1, 2, 4, 8)
            assert p.m_blocks * 16 * p.row_tiles >= M
        assert p.block == 64 * p.waves_n * p.waves_k and p.block <= 1024
        assert p.grid_x * 64 * p.waves_n >= N
        kstep = 32 if bits == 4 else 128
        steps = (K + kstep - 1) // kstep
        assert 1 <= p.split_k <= steps
        assert p.lds_bytes <= 160 * 1024
        assert p.grid_x >= 1 and p.grid_y >= 1 and p.grid_z >= 1
        if p.split_k > 1:
            assert p.workspace_bytes >= p.split_k * M * N * 4
            if p.kernel == _lib.KERNEL_GROUPED and M > 2:   # packed rows: partial sums of all the plan's rows
                assert p.workspace_bytes >= p.split_k * p.row_tiles * N * 4
            # partial sums stay in proportion to the packed weights (or there is a single split)
            assert p.split_k * M * N * 4 <= 3 * K * N * bits // 8 or p.split_k == 2
        elif p.kernel == _lib.KERNEL_STREAM:
            # holds the packed x (at least one 16-row tile over all of K), except for one row
            # tile, where the kernel may read x itself
            assert p.workspace_bytes >= 16 * K * 2 or (p.row_tiles == 1 and p.workspace_bytes == 0)
        else:
            assert p.workspace_bytes == 0
        lib = _lib.lib()
        assert lib.gptq_hip_workspace_bytes(M, K, N, bits, gs, int(act)) == p.workspace_bytes


def test_select_spreads_decode_shapes_over_the_chip():
    # the headline shapes must give most of the 256 CUs a workgroup
    for bits in (3, 4):
        for (K, N) in [(4096, 4096), (4096, 11008), (11008, 4096)]:
            p = _lib.select(1, K, N, bits, 128, True)
            assert p.grid_x * p.grid_y * p.grid_z >= 128, (bits, K, N, p.as_dict())
    # contiguous groups and K <= 4096: one workgroup per column tile even when that leaves CUs idle (a
    # workgroup's time is a chain of load latencies, and the sum across workgroups costs more than it saves)
    for bits in (3, 4):
        for N in (512, 4096):
            p = _lib.select(1, 4096, N, bits, 128, False)
            assert p.kernel == _lib.KERNEL_GROUPED and p.split_k == 1 and p.grid_x == N // 64 and p.workspace_bytes == 0
        assert _lib.select(1, 11008, 4096, bits, 128, False).split_k > 1
    # 4096 x 11008 with 32 groups: one workgroup per 64 columns owns all of K, nothing crosses workgroups
    p = _lib.select(1, 4096, 11008, 3, 128, True)
    assert p.kernel == _lib.KERNEL_GROUPED and p.split_k == 1 and p.workspace_bytes == 0 and p.grid_x == 172


@pytest.mark.parametrize("args", [
    (1, 4096, 4096, 2, 128),   # bits
    (1, 4096, 4096, 8, 128),
    (0, 4096, 4096, 4, 128),   # M
    (1, 4100, 4096, 4, 128),   # K % 32
    (1, 4096, 4100, 4, 128),   # N % 32
    (1, 4096, 4096, 4, 0),     # group_size
    (1, 4096, 4096, 4, -5),
])
def test_select_rejects_bad_arguments(args):
    M, K, N, bits, gs = args
    with pytest.raises(_lib.GptqHipError) as e:
        _lib.select(M, K, N, bits, gs, False)
    assert e.value.status == _lib.ERR_BAD_ARG


def test_entry_points_reject_null_and_bad_sizes_before_touching_the_gpu():
    lib = _lib.lib()
    null = ctypes.c_void_p(None)
    fake = ctypes.c_void_p(0x1000)  # aligned, never dereferenced: the checks fail first
    # null pointers
    assert lib.gptq_hip_gemm(null, fake, fake, fake, null, null, fake, null, 0, 1, 64, 64, 4, 32, null) == _lib.ERR_BAD_ARG
    assert lib.gptq_hip_gemm(fake, null, fake, fake, null, null, fake, null, 0, 1, 64, 64, 4, 32, null) == _lib.ERR_BAD_ARG
    # bits outside {3, 4}
    assert lib.gptq_hip_gemm(fake, fake, fake, fake, null, null, fake, null, 0, 1, 64, 64, 8, 32, null) == _lib.ERR_BAD_ARG
    # K not a multiple of 32
    assert lib.gptq_hip_gemm(fake, fake, fake, fake, null, null, fake, null, 0, 1, 72, 64, 4, 8, null) == _lib.ERR_BAD_ARG
    # misaligned qweight
    assert lib.gptq_hip_gemm(fake, ctypes.c_void_p(0x1004), fake, fake, null, null, fake, null, 0, 1, 64, 64, 4, 32,
                             null) == _lib.ERR_BAD_ARG
    # g_idx that is not 16-byte aligned (the kernels read it four entries at a time)
    assert lib.gptq_hip_gemm(fake, fake, fake, fake, ctypes.c_void_p(0x1004), null, fake, null, 0, 1, 64, 64, 4, 32,
                             null) == _lib.ERR_BAD_ARG
    # a STREAM plan for M > 16 always needs the workspace (packed activations)
    assert lib.gptq_hip_gemm(fake, fake, fake, fake, null, null, fake, null, 0, 64, 4096, 11008, 4, 128,
                             null) == _lib.ERR_WORKSPACE
    # a split-K plan without a workspace
    assert _lib.select(1, 11008, 4096, 4, 128, False).split_k > 1
    assert lib.gptq_hip_gemm(fake, fake, fake, fake, null, null, fake, null, 0, 1, 11008, 4096, 4, 128,
                             null) == _lib.ERR_WORKSPACE
    # packed rows with K split: the partial sums are indexed by the rows the plan is sized for (4 or 8), so a
    # workspace sized for the real M is refused
    pk = _lib.plan_for(_lib.KERNEL_GROUPED, 2, 2048, 320, 4, 128, False, split_k=2)
    pk3 = _lib.plan_for(_lib.KERNEL_GROUPED, 3, 2048, 320, 4, 128, False, split_k=2)
    for M, pl in ((3, pk3),):
        assert pl.row_tiles == 4 and pl.split_k == 2
        small = 16384 + pl.split_k * M * 320 * 4
        assert small < pl.workspace_bytes
        assert lib.gptq_hip_gemm_plan(fake, fake, fake, fake, null, null, fake, fake, small, M, 2048, 320, 4, 128,
                                      ctypes.byref(pl), null) == _lib.ERR_WORKSPACE
    del pk
    # a hand-edited STREAM plan: one row tile but several M blocks (the kernel that reads x itself covers 16 rows)
    ps = _lib.plan_for(_lib.KERNEL_STREAM, 16, 4096, 352, 4, 128, False)
    assert ps.row_tiles == 1 and ps.m_blocks == 1
    ps.m_blocks, ps.grid_z = 2, 2
    assert lib.gptq_hip_gemm_plan(fake, fake, fake, fake, null, null, fake, fake, 1 << 24, 32, 4096, 352, 4, 128,
                                  ctypes.byref(ps), null) == _lib.ERR_BAD_ARG
    # the sorted entry: no map, a misaligned map, a shape outside the decode family, K past the map's 16-bit positions,
    # groups that are not whole lane blocks
    srt = lib.gptq_hip_gemm_sorted
    assert srt(fake, fake, fake, fake, null, null, fake, null, 0, 1, 4096, 11008, 3, 128, None, null) == _lib.ERR_BAD_ARG
    assert srt(fake, fake, fake, fake, ctypes.c_void_p(0x1004), null, fake, null, 0, 1, 4096, 11008, 3, 128, None,
               null) == _lib.ERR_BAD_ARG
    # a small batch runs behind a pass that reorders x into the workspace: none given
    assert srt(fake, fake, fake, fake, fake, null, fake, null, 0, 8, 4096, 11008, 3, 128, None, null) == _lib.ERR_WORKSPACE
    assert srt(fake, fake, fake, fake, fake, null, fake, null, 0, 17, 4096, 11008, 3, 128, None, null) == _lib.ERR_UNSUPPORTED
    assert lib.gptq_hip_sorted_workspace_bytes(8, 4096, 11008, 3, 128) == 16384 + 8 * 4096 * 2   # behind the counters
    assert lib.gptq_hip_sorted_workspace_bytes(1, 4096, 11008, 3, 128) == 0
    p4 = _lib.select(4, 11008, 4096, 4, 128, False)
    assert lib.gptq_hip_sorted_workspace_bytes(4, 11008, 4096, 4, 128) == (max(p4.workspace_bytes, 16384) + 255) // 256 * 256 + 4 * 11008 * 2
    assert srt(fake, fake, fake, fake, fake, null, fake, null, 0, 1, 65536, 64, 4, 128, None, null) == _lib.ERR_UNSUPPORTED
    assert srt(fake, fake, fake, fake, fake, null, fake, null, 0, 1, 4096, 64, 3, 16, None, null) == _lib.ERR_UNSUPPORTED
    # the load-time sort: in place, missing buffers, limits of the map
    assert lib.gptq_hip_sort_channels(fake, fake, fake, fake, 4096, 64, 4, 128, null) == _lib.ERR_BAD_ARG
    assert lib.gptq_hip_sort_channels(fake, fake, null, fake, 4096, 64, 4, 128, null) == _lib.ERR_BAD_ARG
    other = ctypes.c_void_p(0x2000)
    assert lib.gptq_hip_sort_channels(fake, fake, other, fake, 65536, 64, 4, 128, null) == _lib.ERR_UNSUPPORTED
    assert lib.gptq_hip_sort_channels(fake, fake, other, fake, 4096, 64, 3, 16, null) == _lib.ERR_UNSUPPORTED
    assert lib.gptq_hip_sort_channels(fake, fake, other, fake, 4096, 64, 2, 128, null) == _lib.ERR_BAD_ARG
    assert lib.gptq_hip_dequant(fake, fake, fake, null, null, 64, 64, 4, 32, null) == _lib.ERR_BAD_ARG
    assert lib.gptq_hip_dequant(fake, fake, fake, null, fake, 64, 64, 5, 32, null) == _lib.ERR_BAD_ARG
    assert lib.gptq_hip_workspace_init(null, 64, null) == _lib.ERR_BAD_ARG
    assert lib.gptq_hip_workspace_init(null, 0, null) == _lib.OK


def test_plan_for_forces_family_split_and_waves():
    with pytest.raises(_lib.GptqHipError) as e:      # family 1 has been retired
        _lib.plan_for(1, 1, 4096, 11008, 3, 128, True, split_k=5, waves_n=2)
    assert e.value.status == _lib.ERR_UNSUPPORTED
    p = _lib.plan_for(_lib.KERNEL_GROUPED, 1, 4096, 11008, 3, 128, True, split_k=8)
    assert p.kernel == _lib.KERNEL_GROUPED and p.split_k == 8 and p.row_tiles == 2
    assert p.waves_n * p.waves_k * 64 == p.block
    # M = 3 is outside the GROUPED family; so are 128 groups under activation order
    with pytest.raises(_lib.GptqHipError) as e:
        _lib.plan_for(_lib.KERNEL_GROUPED, 3, 4096, 4096, 4, 128, True)
    assert e.value.status == _lib.ERR_UNSUPPORTED
    with pytest.raises(_lib.GptqHipError):
        _lib.plan_for(_lib.KERNEL_GROUPED, 1, 4096, 4096, 4, 32, True)
    with pytest.raises(_lib.GptqHipError) as e:
        _lib.plan_for(_lib.KERNEL_GROUPED, 1, 4096, 4096, 4, 128, True, waves_n=3)
    assert e.value.status == _lib.ERR_BAD_ARG


def test_dispatcher_families_by_m():
    # decode: GROUPED; two to four rows on contiguous groups: GROUPED with the rows packed into one operand
    # tile (a plan sized for four rows); under an activation order M = 2 only while one workgroup holds all
    # of K; batches: STREAM, direct up to 16 rows
    assert _lib.select(1, 4096, 11008, 4, 128, True).kernel == _lib.KERNEL_GROUPED
    for bits, m in [(4, 2), (4, 3), (4, 4), (3, 2), (3, 4), (3, 5), (3, 8)]:
        p = _lib.select(m, 4096, 11008, bits, 128, False)
        assert p.kernel == _lib.KERNEL_GROUPED and p.row_tiles == (4 if m <= 4 else 8) and p.split_k == 1 and p.grid_x == 172
    assert _lib.select(5, 4096, 11008, 4, 128, False).kernel == _lib.KERNEL_STREAM   # two tiles: int3 only
    assert _lib.select(9, 4096, 11008, 3, 128, False).kernel == _lib.KERNEL_STREAM
    # ... unless K would be cut into four or more ranges
    assert _lib.select(4, 11008, 4096, 4, 128, False).kernel == _lib.KERNEL_STREAM
    assert _lib.select(4, 4096, 11008, 4, 128, True).kernel == _lib.KERNEL_STREAM
    p = _lib.select(8, 4096, 11008, 4, 128, True)
    assert p.kernel == _lib.KERNEL_STREAM and p.row_tiles == 1 and p.workspace_bytes == 0 and p.split_k == 1
    p = _lib.select(128, 4096, 11008, 3, 128, True)
    assert p.kernel == _lib.KERNEL_STREAM and p.row_tiles == 4 and p.m_blocks == 2 and p.split_k == 1
    assert p.workspace_bytes >= 128 * 4096 * 2
    # activation order over many groups: past 48 the expansion by group loses to STREAM's lookups, while
    # the same layer with its channels sorted at load is a plain GROUPED problem
    assert _lib.select(1, 11008, 4096, 4, 128, True).kernel == _lib.KERNEL_STREAM
    assert _lib.select(1, 5120, 4096, 3, 128, True).kernel == _lib.KERNEL_GROUPED
    assert _lib.select(1, 11008, 4096, 4, 128, False).kernel == _lib.KERNEL_GROUPED
    # very wide layers: 256 columns per workgroup (four waves along N) keep the grid to one round
    p = _lib.select(1, 9216, 36864, 3, -1, False)
    assert p.kernel == _lib.KERNEL_GROUPED and p.waves_n == 4 and p.grid_x == 144 and p.split_k == 1
    # a GROUPED plan that would cut K into eight or more ranges loses to STREAM's own pass
    assert _lib.select(1, 36864, 9216, 4, -1, False).kernel == _lib.KERNEL_STREAM
    assert _lib.select(1, 36864, 9216, 3, -1, False).kernel == _lib.KERNEL_GROUPED
    # wide workgroups only where they do not force a finer split of K
    assert _lib.select(1, 8192, 28672, 4, 128, False).waves_n == 2
    assert _lib.select(1, 8192, 28672, 3, 128, False).waves_n == 1
    # forcing the STREAM family with waves along K and a split
    p = _lib.plan_for(_lib.KERNEL_STREAM, 40, 4096, 352, 3, 128, True, split_k=2, waves_n=8)
    assert p.kernel == _lib.KERNEL_STREAM and p.waves_k == 8 and p.waves_n == 1 and p.split_k == 2 and p.block == 512
    # more groups than the LDS table of STREAM holds: no fused kernel on the checkpoint layout
    with pytest.raises(_lib.GptqHipError) as e:
        _lib.select(4, 36864, 9216, 4, 32, True)
    assert e.value.status == _lib.ERR_UNSUPPORTED


def test_single_group_ignores_act_order():
    a = _lib.select(1, 9216, 9216, 3, -1, True).as_dict()
    b = _lib.select(1, 9216, 9216, 3, -1, False).as_dict()
    assert a == b


def test_torch_operator_library_is_built_and_matches_the_kernel_library():
    """csrc/binding.cpp: built beside the kernel library, from the same sources (one build id), and it
    defines every operator the module calls, with the schemas the Python front end has."""
    import torch

    from autogptq.tvm_amd import ops

    assert os.path.exists(ops.BINDING_PATH), "run python -m autogptq.tvm_amd.build"
    assert ops.NATIVE_OPS
    assert torch.ops.gptq_hip.binding_build_id() == _lib.build_id()
    for name in ("gemm", "gemm_sorted", "gemm_tiled", "dequant"):
        schema = str(getattr(torch.ops.gptq_hip, name).default._schema)
        assert schema.startswith(f"gptq_hip::{name}(Tensor ") and schema.endswith("-> Tensor"), schema
    assert hasattr(torch.classes.gptq_hip, "Layer")
    # shape-only versions for tracing
    m = torch.ops.gptq_hip.gemm_tiled(torch.empty(5, 64, dtype=torch.float16, device="meta"),
                                      torch.empty(64 * 32 // 8, dtype=torch.int32, device="meta"),
                                      torch.empty(1, 32, dtype=torch.int32, device="meta"), None, None, None, 4, 64)
    assert m.shape == (5, 32) and m.device.type == "meta"


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("KN", [(4096, 4096), (4096, 11008), (11008, 4096), (96, 32), (9216, 36864)])
def test_tiled_plans_are_consistent(bits, KN):
    """The tiled family plans every width of the format; the launches it describes cover the problem and stay
    within a workgroup's LDS (no GPU needed: the plans are host arithmetic)."""
    K, N = KN
    gs = 128 if K % 128 == 0 else 32
    blocks = -(-K // 64)
    for M in (1, 2, 4, 5, 8, 9, 16, 17, 128, 129, 1024):
        p = _lib.select_tiled(M, K, N, bits, gs)
        assert p.lds_bytes <= 160 * 1024 and p.block in (256, 512, 1024) and p.split_k == p.grid_y >= 1
        if M <= 4 or (M <= 8 and K <= 11008):
            assert p.kernel == _lib.KERNEL_TILED_DECODE and p.row_tiles >= M
            if M > 4:                # five to eight rows: the workgroup-per-tile kernel only, at most eight waves
                assert p.row_tiles == 8 and p.waves_n == 1 and p.waves_k in (4, 8)
            if p.waves_n == 2:       # a workgroup per CU, 16-column units, sixteen waves over the 128-position blocks
                assert p.block == 1024 and 1 <= p.grid_x <= min(N // 16, 256) and p.k_chunk * 16 >= -(-blocks // 2)
            else:                    # a workgroup per 32-column tile
                tiles = N // 32
                # (the tiles past a whole number per CU, when there are at most 128 of them, run as two halves
                # along K, which meet in 64-bit slots behind the counters of the workspace)
                # (and every tile of a long layer of up to 4096 columns: two workgroups per tile still find a CU each)
                halved = p.grid_x - tiles
                assert halved in (0, tiles % 256, tiles) and p.split_k * p.waves_k * p.k_chunk >= blocks
                if halved == tiles:
                    assert 2 * tiles <= 256 and blocks >= 64 and p.split_k == 1 and p.waves_k == 8
                elif halved:
                    assert tiles > 256 and halved <= 128 and p.split_k == 1
                if halved:
                    pairs = (K if gs == -1 else gs) % 128 == 0 and p.k_chunk % 2 == 0
                    first = 2 * ((p.k_chunk + 3) // 4) if pairs else (p.k_chunk + 1) // 2
                    assert p.k_chunk - first >= (2 if pairs else 1) and p.waves_k * first < blocks
                    assert p.workspace_bytes == 16384 + halved * p.row_tiles * 32 * 8
                elif p.split_k == 1:
                    assert p.workspace_bytes == 0
        else:
            assert p.kernel == _lib.KERNEL_TILED
            cols = 64 * p.waves_n
            assert p.grid_x * cols >= N and p.grid_z == p.m_blocks and p.m_blocks * p.row_tiles * 32 >= M
            assert p.split_k * p.waves_k * p.k_chunk >= blocks
            assert p.workspace_bytes >= p.split_k * p.waves_k * p.k_chunk * 4 * p.row_tiles * p.m_blocks * 1024
    assert _lib.lib().gptq_hip_tiled_bytes(K, N, bits) == blocks * 64 * N * bits // 8


def test_tiled_plans_reject_what_the_format_does_not_cover():
    for args, status in [((1, 4096, 4096, 5, 128), _lib.ERR_BAD_ARG),      # a width the format does not have
                         ((1, 4096, 4096, 4, 16), _lib.ERR_UNSUPPORTED),   # groups narrower than a lane block
                         ((1, 4096, 4100, 4, 128), _lib.ERR_BAD_ARG),
                         ((0, 4096, 4096, 4, 128), _lib.ERR_BAD_ARG)]:
        with pytest.raises(_lib.GptqHipError) as e:
            _lib.select_tiled(*args)
        assert e.value.status == status, args
    with pytest.raises(_lib.GptqHipError):
        _lib.select_tiled(9, 4096, 4096, 8, 128, decode=True)             # the decode kernels take up to eight rows
    p8 = _lib.select_tiled(5, 4096, 4096, 8, 128, decode=True)            # five to eight: the workgroup-per-tile kernel, two row sets
    assert p8.kernel == _lib.KERNEL_TILED_DECODE and p8.row_tiles == 8 and p8.waves_n == 1 and p8.waves_k in (4, 8)
    assert _lib.lib().gptq_hip_tiled_bytes(4096, 4096, 5) == 0


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("KN", [(4096, 4096), (4096, 11008), (11008, 4096), (96, 32), (9216, 36864), (352, 65536)])
def test_transposed_plans_are_consistent(bits, KN):
    """The plans of the transposed product gx[M, K] = gy[M, N] @ W^T: the grid covers the K columns of the result,
    the waves cover the N columns of the reduction, and the table of a workgroup's range fits its LDS."""
    K, N = KN
    gs = 128 if K % 128 == 0 else 32
    blocks = -(-N // 64)
    for M in (1, 5, 33, 128, 129, 1024):
        p = _lib.select_tiled_transposed(M, K, N, bits, gs)
        assert p.kernel == _lib.KERNEL_TILED and p.waves_n == 1 and p.waves_k == 4 and p.block == 256
        assert p.grid_x == -(-(K // 32) // 2) and p.grid_z == p.m_blocks and p.m_blocks * p.row_tiles * 32 >= M
        assert p.split_k == p.grid_y >= 1 and p.split_k * p.waves_k * p.k_chunk >= blocks
        assert 2 * p.waves_k * p.k_chunk * 256 <= p.lds_bytes <= 160 * 1024
        assert p.lds_bytes >= p.waves_k * p.row_tiles * 2 * 4096
        part = (p.split_k * M * K * 4 + 255) // 256 * 256 if p.split_k > 1 else 0
        assert p.workspace_bytes >= 16384 + part + p.split_k * p.waves_k * p.k_chunk * 4 * p.row_tiles * p.m_blocks * 1024
    lib = _lib.lib()
    assert lib.gptq_hip_tiled_transposed_bytes(K, N, bits) == K * blocks * 64 * bits // 8
    assert lib.gptq_hip_tiled_transposed_table_bytes(K, N, gs) == (K // gs) * blocks * 256
    with pytest.raises(_lib.GptqHipError):
        _lib.select_tiled_transposed(1, K, N, bits, 16)


# ---- which copy a call runs on (gptq_hip_select_route)
def table_tiled_wins(M, K, N, act_order, bits, one_group):
    """The measured table the route rule was written from, stated once more as data-like branches: which row
    counts and shapes the tiled copy won at (group size 128 or one group)."""
    if M <= 4:
        if N <= 4096:
            return True
        if K <= 4096:
            return M <= 2 or N < 16384
        if M <= 2:
            return True
        return K <= 6656 or (K <= 11008 and N <= 8192)
    if M <= 8 and K <= 11008:
        return True
    if M <= 16:
        if not act_order and K > 4096:
            return N > 4096 and not 6656 < K < 11008
        if not act_order:
            return K <= 4096 and N > 4096 and (M >= 9 or bits == 4)
        return K <= 4096 and ((N > 4096 and M >= 12) or (bits == 3 and N <= 4096))
    if M <= 128:
        if one_group and K > 8192 and N > 16384:
            return False
        return not (M <= 64 and K >= 8192 and N >= 8192 and bits == 4 and not act_order)
    return K <= 8192 or (M <= 256 and (K <= 11008 or act_order or (one_group and N <= 16384)))


ROUTE_SHAPES = [(4096, 4096), (4096, 11008), (11008, 4096), (4096, 22016), (8192, 8192), (8192, 28672), (28672, 8192),
                (9216, 9216), (9216, 36864), (36864, 9216), (18432, 9216), (5120, 13824), (6656, 17920), (17920, 6656)]


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("KN", ROUTE_SHAPES)
def test_route_follows_the_measured_table(bits, KN):
    K, N = KN
    for gs in (128, -1):
        if gs == 128 and K % 128 != 0:
            continue
        one_group = gs == -1
        for act in (False, True):
            for M in (1, 2, 3, 4, 5, 8, 9, 16, 17, 32, 33, 64, 65, 128, 129, 256, 639, 640, 1023, 1024, 1151, 1152, 4096):
                r = _lib.select_route(M, K, N, bits, gs, act)
                act_eff = act and not one_group
                tiled = table_tiled_wins(M, K, N, act_eff, bits, one_group)
                limit = 1152 if tiled else (640 if act_eff else 1024)
                if M >= limit:
                    assert r.copy == _lib.ROUTE_LIBRARY and r.plan.kernel == 0, (M, K, N, gs, act)
                    continue
                if tiled:
                    assert r.copy == _lib.ROUTE_TILED, (M, K, N, gs, act)
                    assert r.plan.as_dict() == _lib.select_tiled(M, K, N, bits, gs).as_dict()
                    continue
                assert r.copy in (_lib.ROUTE_SORTED, _lib.ROUTE_CHECKPOINT, _lib.ROUTE_LIBRARY), (M, K, N, gs, act)
                if r.copy == _lib.ROUTE_SORTED:
                    assert act_eff and M <= 16
                    assert r.plan.as_dict() == _lib.select(M, K, N, bits, gs, False).as_dict()
                elif r.copy == _lib.ROUTE_CHECKPOINT:
                    assert r.plan.as_dict() == _lib.select(M, K, N, bits, gs, act_eff).as_dict()


def test_route_honours_the_copies_on_offer_and_the_switch_rows():
    K, N = 4096, 11008
    # a layer that keeps only its tiled copy: every row count runs there, whatever the switch says
    for M in (1, 8, 128, 5000):
        r = _lib.select_route(M, K, N, 4, 128, True, copies=_lib.COPY_TILED)
        assert r.copy == _lib.ROUTE_TILED and r.plan.kernel in (_lib.KERNEL_TILED, _lib.KERNEL_TILED_DECODE)
    # without the tiled copy: decode sizes of an activation-order layer on the sorted copy, the rest on the checkpoint
    no_tiled = _lib.COPY_CHECKPOINT | _lib.COPY_SORTED
    assert _lib.select_route(1, K, N, 3, 128, True, copies=no_tiled).copy == _lib.ROUTE_SORTED
    assert _lib.select_route(1, K, N, 3, 128, False, copies=no_tiled).copy == _lib.ROUTE_CHECKPOINT
    assert _lib.select_route(64, K, N, 3, 128, True, copies=no_tiled).copy == _lib.ROUTE_CHECKPOINT
    assert _lib.select_route(1, K, N, 3, 128, True, copies=_lib.COPY_CHECKPOINT).copy == _lib.ROUTE_CHECKPOINT
    # 2 and 8 bits: fused on the tiled copy only
    assert _lib.select_route(1, K, N, 8, 128, True).copy == _lib.ROUTE_TILED
    assert _lib.select_route(1, K, N, 8, 128, True, copies=no_tiled).copy == _lib.ROUTE_LIBRARY
    # groups the tiled format does not cover stay off it
    assert _lib.select_route(64, K, N, 4, 16, False).copy == _lib.ROUTE_CHECKPOINT
    # switch rows: the caller's, 0 = never
    assert _lib.select_route(128, K, N, 4, 128, True, switch_rows=(128, 128, 128)).copy == _lib.ROUTE_LIBRARY
    assert _lib.select_route(127, K, N, 4, 128, True, switch_rows=(128, 128, 128)).copy == _lib.ROUTE_TILED
    assert _lib.select_route(100000, K, N, 4, 128, True, switch_rows=(0, 0, 0)).copy == _lib.ROUTE_TILED
    # more activation-order groups than any fused kernel on the checkpoint layout takes
    assert _lib.select_route(4, 36864, 9216, 4, 32, True, copies=_lib.COPY_CHECKPOINT).copy == _lib.ROUTE_LIBRARY
    with pytest.raises(_lib.GptqHipError):
        _lib.select_route(1, K, N, 4, 128, True, copies=0)
    with pytest.raises(_lib.GptqHipError):
        _lib.select_route(1, K, N, 5, 128, True)
    with pytest.raises(_lib.GptqHipError):
        _lib.select_route(0, K, N, 4, 128, True)


def test_plans_that_need_a_private_zero_workspace_say_so():
    # halved tiles of the decode kernel meet in slots of the workspace: the plan carries the flag, others do not
    p = _lib.select_tiled(1, 4096, 11008, 3, 128)
    assert p.kernel == _lib.KERNEL_TILED_DECODE and p.grid_x > 11008 // 32
    assert p.flags & _lib.PLAN_PRIVATE_ZERO_WORKSPACE and p.workspace_bytes > 0
    q = _lib.select_tiled(1, 4096, 4096, 4, 128)     # every tile of a narrow layer of 4096 channels and more in two halves
    assert q.kernel == _lib.KERNEL_TILED_DECODE and q.waves_n == 1 and q.grid_x == 2 * (4096 // 32)
    assert q.flags & _lib.PLAN_PRIVATE_ZERO_WORKSPACE and q.workspace_bytes > 0
    for q in (_lib.select_tiled(1, 2048, 4096, 4, 128), _lib.select_tiled(128, 4096, 11008, 4, 128),
              _lib.select(1, 4096, 11008, 3, 128, True), _lib.select(64, 4096, 11008, 4, 128, True)):
        assert q.flags == 0
    assert ctypes.sizeof(_lib.Route) == 8 + ctypes.sizeof(_lib.Plan)


@pytest.mark.parametrize("bits", [3, 4])
def test_plans_of_two_and_four_row_tiles_fill_their_turns_of_the_chip(bits):
    # a workgroup of two or four row tiles holds a CU alone: K ranges never put a few workgroups past a turn of the CUs
    for K, N in ROUTE_SHAPES + [(4096, 6144), (8192, 5632), (4096, 3328), (11008, 11008), (8192, 6144), (11008, 4608)]:
        for M in (33, 64, 97, 128, 192, 256, 512):
            plans = [_lib.select_tiled(M, K, N, bits, 128)]
            if N <= 11008:   # (longer reductions of the transposed product are cut so that a range's table fits LDS)
                plans.append(_lib.select_tiled_transposed(M, K, N, bits, 128))
            for p in plans:
                if p.kernel != _lib.KERNEL_TILED or p.row_tiles < 2:
                    continue
                tiles = p.grid_x * p.grid_z
                assert p.grid_y == p.split_k
                # (whole turns of the 256 CUs, or enough of the last one: never a few workgroups past a turn)
                past = (tiles * p.split_k) % 256
                assert p.split_k == 1 or tiles > 256 or past == 0 or past >= 96, (M, K, N, p.as_dict())


def test_narrow_layers_run_in_shorter_row_blocks():
    # 65 to 256 rows of a narrow layer: blocks of 64 rows while they find a CU each (K up to 8192), 33 to 64 rows as two
    # blocks of 32 (K up to 4096); the wide and the long layers keep the taller blocks
    for M, K, N, rt, mb in ((128, 4096, 4096, 2, 2), (256, 4096, 4096, 2, 4), (192, 5120, 5120, 2, 3), (128, 8192, 8192, 2, 2),
                            (320, 4096, 4096, 4, 3), (256, 5120, 5120, 4, 2), (128, 4096, 11008, 4, 1), (128, 11008, 4096, 4, 1),
                            (64, 4096, 4096, 1, 2), (48, 4096, 8192, 1, 2), (64, 8192, 4096, 2, 1), (64, 4096, 11008, 2, 1),
                            (32, 4096, 4096, 1, 1)):
        p = _lib.select_tiled(M, K, N, 4, 128)
        assert (p.kernel, p.row_tiles, p.m_blocks, p.grid_z) == (_lib.KERNEL_TILED, rt, mb, mb), (M, K, N, p.as_dict())
        assert p.waves_n == 1 or p.row_tiles == 4
        assert p.lds_bytes == 4 * p.row_tiles * 2 * 4096 * (2 if p.waves_n == 2 else 1) or p.waves_n == 2
    p = _lib.select_tiled(128, 4096, 4096, 4, 128)
    assert p.split_k == 1 and p.k_chunk == 16
    p = _lib.select_tiled(128, 8192, 4096, 4, 128)
    assert p.split_k == 2 and p.k_chunk == 16


def test_matmul_plans_keep_the_measured_choices():
    # (M, K, N, bits, group_size) -> (row tiles, row blocks, waves along N, K ranges): the plans that the measurements
    # named as the best of their neighbours on MI355X (the count of turns of the chip and the shorter row blocks of
    # narrow layers); a change of the planner that moves one of them wants a measurement
    table = [
        (128, 36864, 9216, 3, -1, 4, 1, 1, 3), (64, 36864, 9216, 3, -1, 2, 1, 1, 3), (128, 9216, 9216, 3, 128, 4, 1, 1, 1),
        (64, 8192, 6144, 4, 128, 2, 1, 1, 2), (64, 11008, 4608, 4, 128, 2, 1, 1, 3), (64, 8192, 3328, 4, 128, 2, 1, 1, 4),
        (128, 11008, 4096, 4, 128, 4, 1, 1, 4), (256, 11008, 4096, 4, 128, 4, 2, 2, 3), (192, 11008, 4096, 4, 128, 4, 2, 2, 3),
        (128, 4096, 11008, 4, 128, 4, 1, 1, 1), (256, 4096, 11008, 4, 128, 4, 2, 2, 1), (64, 4096, 11008, 3, 128, 2, 1, 1, 1),
        (32, 13824, 5120, 4, 128, 1, 1, 1, 3), (32, 28672, 8192, 4, 128, 1, 1, 1, 2), (32, 4096, 9216, 4, 128, 1, 1, 1, 1),
        (32, 9216, 9216, 3, -1, 1, 1, 1, 3), (32, 36864, 9216, 3, -1, 1, 1, 1, 3), (16, 4096, 11008, 4, 128, 1, 1, 1, 1),
        (128, 4096, 4096, 4, 128, 2, 2, 1, 1), (128, 8192, 4096, 4, 128, 2, 2, 1, 2), (64, 4096, 4096, 4, 128, 1, 2, 1, 1),
        (256, 4096, 4096, 4, 128, 2, 4, 1, 1),
    ]
    for M, K, N, bits, gs, rt, mb, wn, split in table:
        p = _lib.select_tiled(M, K, N, bits, gs)
        assert (p.kernel, p.row_tiles, p.m_blocks, p.waves_n, p.split_k) == (_lib.KERNEL_TILED, rt, mb, wn, split), (
            M, K, N, bits, gs, p.as_dict())
    # the kernels on the checkpoint tensors: K ranges within one workgroup per CU
    for M, K, N, bits, kernel, split in ((1, 8192, 5120, 4, _lib.KERNEL_GROUPED, 3), (1, 8192, 6144, 4, _lib.KERNEL_GROUPED, 2),
                                         (1, 11008, 4096, 4, _lib.KERNEL_GROUPED, 4), (9, 8192, 6144, 4, _lib.KERNEL_STREAM, 2),
                                         (32, 11008, 4608, 4, _lib.KERNEL_STREAM, 3), (16, 11008, 4096, 4, _lib.KERNEL_STREAM, 4)):
        p = _lib.select(M, K, N, bits, 128, False)
        assert (p.kernel, p.split_k) == (kernel, split), (M, K, N, bits, p.as_dict())
        assert p.grid_x * p.grid_y * p.grid_z <= 256
