"""Host-side behaviour of QuantLinear that needs no GPU: constructor contract, buffer names,
meta-device construction, and loud failure when asked to compute off the GPU."""
import pytest
import torch

from autogptq.tvm_amd import QuantLinear, ops


def test_buffers_follow_the_reference_layout():
    q = QuantLinear(3, 128, 4096, 11008, True)
    sd = q.state_dict()
    assert set(sd) == {"qweight", "qzeros", "scales", "g_idx", "bias"}
    assert sd["qweight"].shape == (384, 11008) and sd["qweight"].dtype == torch.int32
    assert sd["qzeros"].shape == (32, 1032) and sd["qzeros"].dtype == torch.int32
    assert sd["scales"].shape == (32, 11008) and sd["scales"].dtype == torch.float16
    assert sd["g_idx"].shape == (4096,) and sd["g_idx"].dtype == torch.int32
    assert sd["g_idx"][127] == 0 and sd["g_idx"][128] == 1
    assert q.maxq == 7 and q.groupsize == 128 and q.infeatures == 4096 and q.outfeatures == 11008
    q = QuantLinear(4, -1, 9216, 9216, False)
    assert q.groupsize == 9216 and q.bias is None
    assert q.scales.shape == (1, 9216) and q.qzeros.shape == (1, 1152)
    assert set(q.state_dict()) == {"qweight", "qzeros", "scales", "g_idx"}


@pytest.mark.parametrize("bits", [1, 5, 16])
def test_unsupported_bits_raise(bits):
    with pytest.raises(NotImplementedError):
        QuantLinear(bits, 128, 256, 256, False)


def test_constructs_on_meta_device_without_touching_a_gpu():
    with torch.device("meta"):
        q = QuantLinear(4, 128, 4096, 4096, True)
    assert q.qweight.is_meta and q.scales.is_meta and q.g_idx.is_meta


def test_state_dict_round_trip():
    a = QuantLinear(4, 32, 64, 32, True)
    a.qweight.random_(0, 1000)
    a.scales.fill_(0.5)
    b = QuantLinear(4, 32, 64, 32, True)
    b.load_state_dict(a.state_dict())
    assert torch.equal(b.qweight, a.qweight) and torch.equal(b.scales, a.scales)


def test_forward_on_cpu_fails_loudly():
    q = QuantLinear(4, 32, 64, 32, False)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        q(torch.zeros(1, 64))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.dequant(q.qweight, q.qzeros, q.scales, None, 4, 32)


def test_shape_checks():
    q = QuantLinear(4, 32, 64, 32, False)
    with pytest.raises(ValueError):
        ops.check_shapes(q.qweight, q.qzeros, q.scales[:, :16], None, None, 4, 32)
    with pytest.raises(ValueError):
        ops.check_shapes(q.qweight, q.qzeros, q.scales, q.g_idx[:10], None, 4, 32)
    with pytest.raises(NotImplementedError):
        ops.check_shapes(q.qweight, q.qzeros, q.scales, None, None, 2, 32)
    assert ops.check_shapes(q.qweight, q.qzeros, q.scales, q.g_idx, None, 4, 32) == (64, 32, 2)


def test_torch_ops_are_registered_without_a_cpu_kernel():
    from autogptq.tvm_amd import ops  # noqa: F401  (registers the operators)

    q = QuantLinear(4, 32, 64, 96, False)
    x = torch.zeros((3, 64), dtype=torch.float16)
    meta = [t.to("meta") for t in (x, q.qweight, q.qzeros, q.scales)]
    y = torch.ops.gptq_hip.gemm(meta[0], meta[1], meta[2], meta[3], None, None, 4, 32)
    assert y.device.type == "meta" and tuple(y.shape) == (3, 96) and y.dtype == torch.float16
    w = torch.ops.gptq_hip.dequant(meta[1], meta[2], meta[3], None, 4, 32)
    assert tuple(w.shape) == (64, 96) and w.dtype == torch.float16
    with pytest.raises((NotImplementedError, RuntimeError)):   # no CPU fallback, not even in the dispatcher
        torch.ops.gptq_hip.gemm(x, q.qweight, q.qzeros, q.scales, None, None, 4, 32)


def test_copies_and_pickles_drop_the_routes():
    """A route holds bound launch objects and closures over the module's tensors; copy.deepcopy, pickle and
    torch.save of a module that has served calls must work (the reference's module is a plain one that does) and
    the copy decides its routes again instead of computing on the original's tensors."""
    import copy
    import io
    import pickle
    import threading

    q = QuantLinear(4, 32, 64, 32, True)
    q.qweight.random_(0, 1 << 20)
    # what a served call leaves behind: the watched buffers, their versions, the path, a callable that cannot be copied
    lock = threading.Lock()
    q._g_state = (("stale",), True)      # (any attribute assignment empties the routes: set this first)
    q._routes[1] = (q._watched(), sum(t._version for t in q._watched()), "plain", lambda x, lock=lock: x)
    for clone in (copy.deepcopy(q), pickle.loads(pickle.dumps(q))):
        assert clone._routes == {} and clone._g_state is None and clone._sorted is None and clone._tiled is None
        assert torch.equal(clone.qweight, q.qweight) and clone.qweight.data_ptr() != q.qweight.data_ptr()
        assert (clone.bits, clone.groupsize, clone.infeatures, clone.outfeatures) == (4, 32, 64, 32)
    buf = io.BytesIO()
    torch.save(torch.nn.Sequential(q), buf)
    assert q._routes                      # the original keeps its routes
    # replacing a buffer behind __setattr__'s back (what offload hooks do) makes a cached route stale
    r = q._routes[1]
    assert q._fresh(r)
    q._buffers["qweight"] = q.qweight.clone()
    assert not q._fresh(r)


def test_find_layers_matches_the_reference_helper_on_a_nested_model():
    """auto_gptq/modeling/_utils.py:38-49: names are dotted paths, depth first in registration order; a module
    that is itself a layer comes back under the given name."""
    from autogptq.tvm_amd.loader import find_layers

    net = torch.nn.Sequential()
    net.add_module("a", torch.nn.Linear(4, 4))
    inner = torch.nn.Module()
    inner.proj = torch.nn.Linear(4, 4)
    inner.act = torch.nn.ReLU()
    inner.conv = torch.nn.Conv2d(1, 1, 1)
    net.add_module("blk", inner)
    net.add_module("z", torch.nn.LayerNorm(4))
    found = find_layers(net)
    assert list(found) == ["a", "blk.proj", "blk.conv"] and found["blk.proj"] is inner.proj
    assert list(find_layers(net, [torch.nn.LayerNorm])) == ["z"]
    assert list(find_layers(inner.proj, name="model.q")) == ["model.q"]
    assert find_layers(torch.nn.ReLU()) == {}
