"""The checkpoint loader (reference: auto_gptq/modeling/_utils.py:38-90, _base.py:478-569)."""
import numpy as np
import pytest
import torch

from autogptq.tvm_amd import QuantLinear
from autogptq.tvm_amd.loader import find_layers, from_quantized, make_quant, pack_model, save_quantized
from tests.loader_util import build_checkpoint


def test_find_layers_and_make_quant_on_a_plain_module():
    net = torch.nn.Sequential()
    net.add_module("a", torch.nn.Linear(64, 32, bias=True))
    net.add_module("act", torch.nn.ReLU())
    inner = torch.nn.Module()
    inner.proj = torch.nn.Linear(32, 64, bias=False)
    net.add_module("inner", inner)
    layers = find_layers(net)
    assert sorted(layers) == ["a", "inner.proj"]
    make_quant(net, ["inner.proj"], 3, 32)
    assert isinstance(net.a, torch.nn.Linear)
    q = net.inner.proj
    assert isinstance(q, QuantLinear) and (q.infeatures, q.outfeatures, q.bits, q.groupsize) == (32, 64, 3, 32)
    assert q.bias is None and q.qweight.shape == (3, 64)
    make_quant(net, ["inner.proj"], 3, 32)  # already quantised: left alone
    assert net.inner.proj is q


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
def test_pack_model_packs_the_quantised_layers_in_place(bits):
    """What the reference does after its GPTQ loop (auto_gptq/modeling/_utils.py:123-157): layers named in
    ``quantizers`` become packed QuantLinear layers, other layers stay as they are.  The float weights here lie
    on the quantisation grid, so packing must find exactly the codes they were made from."""
    from oracle import gptq_oracle

    gen = torch.Generator().manual_seed(40 + bits)
    K, N, gs = 128, 64, 32
    G, maxq = K // gs, 2 ** bits - 1
    g_idx = (torch.randperm(K, generator=gen) // gs).to(torch.int32)       # an activation order
    scale = (torch.rand(N, G, generator=gen) * 9e-3 + 1e-3).half().float()  # [N, G], as the reference passes them
    zero = torch.randint(1, maxq + 2, (N, G), generator=gen).float()        # the format stores zero - 1
    codes = torch.randint(0, maxq + 1, (N, K), generator=gen)
    gl = g_idx.long()
    net = torch.nn.Sequential()
    net.add_module("keep", torch.nn.Linear(K, K))
    net.add_module("q", torch.nn.Linear(K, N, bias=True))
    net.q.weight.data = scale[:, gl] * (codes.float() - zero[:, gl])          # exact in fp32
    packed = pack_model(net, {"q": (None, scale, zero, g_idx)}, bits, gs)
    assert sorted(packed) == ["q"] and isinstance(net.q, QuantLinear) and isinstance(net.keep, torch.nn.Linear)
    q = net.q
    assert (q.bits, q.groupsize, q.infeatures, q.outfeatures) == (bits, gs, K, N) and q.bias is not None
    assert np.array_equal(gptq_oracle.unpack_bitstream(q.qweight.numpy(), bits, axis=0), codes.t().numpy())
    assert np.array_equal(gptq_oracle.unpack_bitstream(q.qzeros.numpy(), bits, axis=1) + 1, zero.t().numpy())
    assert torch.equal(q.g_idx, g_idx) and torch.equal(q.scales, scale.t().half())
    w16 = gptq_oracle.dequant_exact(q.qweight.numpy(), q.qzeros.numpy(), q.scales.numpy(), q.g_idx.numpy(), bits)
    assert np.array_equal(w16, (scale[:, gl] * (codes.float() - zero[:, gl])).t().half().numpy())


def test_make_quant_on_meta_allocates_nothing():
    import accelerate

    with accelerate.init_empty_weights(include_buffers=True):
        net = torch.nn.Sequential(torch.nn.Linear(4096, 11008, bias=False))
        make_quant(net, ["0"], 4, 128)
    assert net[0].qweight.device.type == "meta" and net[0].qweight.shape == (512, 11008)


@pytest.mark.parametrize("bits,act_order", [(4, True), (3, False)])
def test_from_quantized_restores_every_tensor(tmp_path, bits, act_order):
    cfg, state, dense = build_checkpoint(str(tmp_path), bits=bits, gs=32, act_order=act_order)
    model, qcfg = from_quantized(str(tmp_path), device="cpu")
    assert qcfg["bits"] == bits and qcfg["group_size"] == 32
    quantised = {n: m for n, m in model.named_modules() if isinstance(m, QuantLinear)}
    assert len(quantised) == 2 * 7 and "lm_head" not in quantised           # q k v o gate up down per layer
    assert isinstance(model.lm_head, torch.nn.Linear)
    got = model.state_dict()
    for name, want in state.items():
        assert name in got, name
        assert got[name].dtype == want.dtype and got[name].device.type == "cpu", name
        assert torch.equal(got[name], want), name
    assert model.seqlen == 64 and not model.training
    with pytest.raises(RuntimeError):  # no CPU path: the kernels must not be silently replaced
        model(torch.zeros((1, 4), dtype=torch.long))


@pytest.mark.parametrize("use_safetensors", [True, False])
def test_pack_save_load_round_trip(tmp_path, use_safetensors):
    """The reference's whole way from a quantised float model to a loaded checkpoint, on a tiny Llama:
    pack_model (_utils.py:123-157), save_quantized (_base.py:381-401), from_quantized (_base.py:478-569)."""
    from transformers import AutoModelForCausalLM, LlamaConfig

    from tests.loader_util import rtn_quantize

    torch.manual_seed(3)
    bits, gs = 4, 32
    cfg = LlamaConfig(hidden_size=64, intermediate_size=128, num_hidden_layers=1, num_attention_heads=4,
                      num_key_value_heads=4, vocab_size=128, max_position_embeddings=64, tie_word_embeddings=False)
    model = AutoModelForCausalLM.from_config(cfg).half()
    quantizers = {}
    for name, lin in find_layers(model).items():
        if name.startswith("lm_head"):
            continue
        scales, zeros = rtn_quantize(lin.weight.data, bits, gs)
        g_idx = (torch.arange(lin.weight.shape[1]) // gs).to(torch.int32)
        quantizers[name] = (None, scales, zeros, g_idx)
    packed = pack_model(model, quantizers, bits, gs)
    assert len(packed) == 7 and isinstance(model.lm_head, torch.nn.Linear)
    path = save_quantized(model, str(tmp_path), bits, gs, desc_act=False, use_safetensors=use_safetensors)
    assert path.endswith(".safetensors" if use_safetensors else ".bin")
    loaded, qcfg = from_quantized(str(tmp_path), device="cpu", use_safetensors=use_safetensors)
    assert (qcfg["bits"], qcfg["group_size"], qcfg["desc_act"]) == (bits, gs, False)
    want, got = model.state_dict(), loaded.state_dict()
    assert sorted(want) == sorted(got)
    for name in want:
        assert want[name].dtype == got[name].dtype and torch.equal(want[name].cpu(), got[name]), name
    # a layer that kept only its tiled copy has nothing left to save
    q = next(m for m in model.modules() if isinstance(m, QuantLinear))
    q._compact = True
    with pytest.raises(ValueError, match="compact"):
        save_quantized(model, str(tmp_path), bits, gs)


def test_from_quantized_reports_missing_files_and_tensors(tmp_path):
    with pytest.raises(FileNotFoundError):
        from_quantized(str(tmp_path))
    cfg, state, dense = build_checkpoint(str(tmp_path), bits=4, gs=32, act_order=False)
    from safetensors.torch import save_file

    broken = {k: v for k, v in state.items() if not k.endswith("q_proj.qzeros")}
    save_file(broken, str(tmp_path / "gptq_model-4bit-32g.safetensors"))
    with pytest.raises(KeyError):
        from_quantized(str(tmp_path), device="cpu")


@pytest.mark.gpu
@pytest.mark.parametrize("keep", [False, True])
@pytest.mark.parametrize("bits,act_order", [(4, True), (3, True), (4, False), (8, True), (2, False)])
def test_loaded_model_matches_the_dequantised_float_model(tmp_path, bits, act_order, keep):
    """End to end: logits of the loaded quantised model on the GPU against the same architecture
    with every quantised layer replaced by a float Linear holding the oracle's dequantised weight."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from transformers import AutoModelForCausalLM

    from oracle import gptq_oracle as orc

    cfg, state, dense = build_checkpoint(str(tmp_path), bits=bits, gs=32, act_order=act_order, seed=3)
    model, _ = from_quantized(str(tmp_path), device="cuda:0", keep_checkpoint_tensors=keep)
    assert all(m._compact != keep for m in model.modules() if isinstance(m, QuantLinear))
    ref = AutoModelForCausalLM.from_config(cfg).float()
    ref_state = {}
    for k, v in state.items():
        if k.endswith((".qweight", ".qzeros", ".scales", ".g_idx")):
            continue
        ref_state[k] = v.float()
    for name, q in dense.items():
        w = orc.dequant_ref(q.qweight, q.qzeros, q.scales, q.g_idx, bits)   # [K, N] fp16
        ref_state[name + ".weight"] = w.t().float().contiguous()
    ref.load_state_dict(ref_state, strict=True)
    ref.eval()
    ids = torch.randint(0, cfg.vocab_size, (2, 9), generator=torch.Generator().manual_seed(5))
    with torch.no_grad():
        want = ref(ids).logits
        got = model(ids.to("cuda:0")).logits.float().cpu()
    assert got.shape == want.shape
    # fp16 activations through two decoder layers against an fp32 model
    assert float((got - want).abs().max()) <= 2e-2 + 2e-2 * float(want.abs().max())
    assert np.isfinite(got.numpy()).all()


def layer_device_bytes(q):
    """Bytes of device memory a QuantLinear holds: its buffers and whatever prepared copies it keeps."""
    seen, total = set(), 0
    held = [q.qweight, q.qzeros, q.scales, q.g_idx, q.bias]
    for slot in (q._sorted, q._tiled, q._tiled_t):
        if slot is not None and slot[1] is not None:
            held += list(slot[1])
    for t in held:
        if t is None or t.device.type != "cuda" or t.data_ptr() in seen:
            continue
        seen.add(t.data_ptr())
        total += t.numel() * t.element_size()
    return total


@pytest.mark.gpu
@pytest.mark.parametrize("bits,act_order", [(4, True), (3, True), (4, False)])
def test_loaded_layers_hold_one_copy_of_their_weights(tmp_path, bits, act_order):
    """After from_quantized and calls with 1, 8 and 128 rows, a layer holds its packed size and the small tables
    (scale / zero words, channel maps), not a second or third copy; nothing is allocated for it by the calls."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    build_checkpoint(str(tmp_path), bits=bits, gs=32, act_order=act_order, seed=8)
    model, _ = from_quantized(str(tmp_path), device="cuda:0")
    layers = {n: m for n, m in model.named_modules() if isinstance(m, QuantLinear)}
    assert layers
    before = {n: layer_device_bytes(m) for n, m in layers.items()}
    for rows in (1, 8, 128):
        for m in layers.values():
            m(torch.randn(rows, m.infeatures, dtype=torch.float16, device="cuda:0"))
    torch.cuda.synchronize()
    for n, m in layers.items():
        K, N, G = m.infeatures, m.outfeatures, m.infeatures // m.groupsize
        packed = K * N * bits // 8
        tables = G * N * 4 + 6 * K + (2 * N if m.bias is not None else 0) + 4 * K   # sz, xsrc + kinv, bias, g_idx
        assert layer_device_bytes(m) == before[n], n
        assert before[n] <= 1.05 * packed + tables, (n, before[n], packed, tables)
