"""The entry point that allocates nothing (gptq_hip_gemm_static) against gptq_hip_gemm on the same inputs:
same kernels, same plan, so the outputs must be bit-equal; two calls in a row, the second smaller."""
import ctypes

import pytest
import torch

from autogptq.tvm_amd import _lib, ops
from tests.parity_util import assert_close, expected_output, layer, to_dev

pytestmark = pytest.mark.gpu


def _static(D, M):
    dev = D["x"].device
    y = torch.full((M, D["N"]), float("nan"), dtype=torch.float16, device=dev)
    vp = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())
    g = D["g_idx"] if D["desc_act"] else None
    rc = _lib.lib().gptq_hip_gemm_static(vp(D["x"]), vp(D["qweight"]), vp(D["qzeros"]), vp(D["scales"]), vp(g),
                                         vp(D.get("bias")), vp(y), M, D["K"], D["N"], D["bits"], D["group_size"],
                                         ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
    return rc, y


# (bits, K, N, gs, desc_act, M): plans that use the workspace -- packed activations (M > 16), split-K with a reduce
# pass, split-K with counters -- first a larger problem, then a smaller one on the same array
CASES = [
    [(4, 4096, 1056, 128, True, 130), (4, 2048, 320, 128, True, 20)],
    [(3, 11008, 4096, 128, False, 1), (3, 8192, 352, 128, False, 1)],
    [(4, 11008, 4096, 128, True, 8), (3, 4096, 352, 128, True, 40)],
]


@pytest.mark.parametrize("pair", CASES, ids=["packed-x", "split-k-counters", "split-k-reduce"])
def test_static_entry_matches_the_allocating_one(pair):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    dev = torch.device("cuda:0")
    assert _lib.lib().gptq_hip_static_workspace_limit() == 16 << 20
    for bits, K, N, gs, act, M in pair:
        L = layer(8100 + M + K, K, N, bits, gs, act, M=M, bias=True)
        D = to_dev(L, dev)
        D.update(K=K, N=N)
        plan = _lib.select(M, K, N, bits, gs, act)
        assert plan.workspace_bytes > 0, "the case is meant to exercise the scratch array"
        want = ops.gemm(D["x"], D["qweight"], D["qzeros"], D["scales"], D["g_idx"] if act else None, D["bias"], bits, gs)
        rc, got = _static(D, M)
        assert rc == _lib.OK
        assert torch.equal(got, want), f"static entry differs from gptq_hip_gemm at {(bits, K, N, gs, act, M)}"
        assert_close(got, expected_output(L), "static entry vs oracle")
        rc2, again = _static(D, M)      # the array keeps the last call's contents: the counters must be back at zero
        assert rc2 == _lib.OK and torch.equal(again, want)


def test_static_entry_rejects_what_the_array_cannot_hold():
    # M = 4096 rows of packed activations need far more than 16 MiB: refused before anything is launched
    lib = _lib.lib()
    plan = _lib.select(4096, 4096, 11008, 4, 128, True)
    assert plan.workspace_bytes > lib.gptq_hip_static_workspace_limit()
    fake, null = ctypes.c_void_p(0x1000), ctypes.c_void_p(None)
    assert lib.gptq_hip_gemm_static(fake, fake, fake, fake, fake, null, fake, 4096, 4096, 11008, 4, 128, null) == _lib.ERR_WORKSPACE


def test_static_entry_replays_from_a_captured_graph():
    """What the entry point is for: a call recorded into a HIP graph (no allocation, no fill, no lookup inside the
    capture once gptq_hip_static_init has run), replayed several times with eager work in between; every replay
    must equal the eager result."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    dev = torch.device("cuda:0")
    assert _lib.lib().gptq_hip_static_init() == _lib.OK
    bits, K, N, gs, act, M = 4, 4096, 1056, 128, True, 40
    L = layer(8200, K, N, bits, gs, act, M=M, bias=True)
    D = to_dev(L, dev)
    D.update(K=K, N=N)
    want = ops.gemm(D["x"], D["qweight"], D["qzeros"], D["scales"], D["g_idx"], D["bias"], bits, gs)
    y = torch.zeros((M, N), dtype=torch.float16, device=dev)
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = torch.cuda.Stream(device=dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        rc = _lib.lib().gptq_hip_gemm_static(vp(D["x"]), vp(D["qweight"]), vp(D["qzeros"]), vp(D["scales"]), vp(D["g_idx"]),
                                             vp(D["bias"]), vp(y), M, K, N, bits, gs,
                                             ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
    assert rc == _lib.OK
    for rep in range(3):
        y.zero_()
        torch.cuda.synchronize(dev)
        graph.replay()
        torch.cuda.synchronize(dev)
        assert torch.equal(y, want), f"replay {rep} differs from the eager result"
        # eager work of the program's own between the replays, on the same array
        rc2, eager = _static(D, M)
        assert rc2 == _lib.OK and torch.equal(eager, want)
