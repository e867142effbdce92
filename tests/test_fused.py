"""Layers that share an input fused into one product (q/k/v, gate/up: the groups of
auto_gptq/modeling/llama.py:8-12)."""
import numpy as np
import pytest
import torch

from autogptq.tvm_amd import QuantLinear, fused
from autogptq.tvm_amd.pack import synth_layer
from oracle import gptq_oracle as orc
from tests.loader_util import build_checkpoint


def member(seed, K, N, bits, gs, g_idx=None, bias=True):
    L = synth_layer(seed, K, N, bits, gs, True, M=3, bias=bias)
    q = QuantLinear(bits, gs, K, N, bias)
    if g_idx is not None:
        # regroup: the codes stay, the scales/zeros rows are now looked up through the shared g_idx
        L["g_idx"] = g_idx
    q.load_state_dict({k: L[k] for k in ("qweight", "qzeros", "scales", "g_idx") + (("bias",) if bias else ())})
    return q, L


@pytest.mark.parametrize("bits", [3, 4])
def test_concat_represents_the_concatenated_weight(bits):
    K, gs = 256, 64
    q1, L1 = member(1, K, 64, bits, gs)
    q2, _ = member(2, K, 96, bits, gs, g_idx=L1["g_idx"])
    q3, _ = member(3, K, 32, bits, gs, g_idx=L1["g_idx"])
    f = fused.concat_qlinears([q1, q2, q3])
    assert (f.infeatures, f.outfeatures, f.bits, f.groupsize) == (K, 192, bits, gs)
    assert f.qweight.shape == (K // 32 * bits, 192) and f.qzeros.shape == (K // gs, 192 // 32 * bits)
    w = orc.dequant_ref(f.qweight, f.qzeros, f.scales, f.g_idx, bits)
    parts = [orc.dequant_ref(q.qweight, q.qzeros, q.scales, q.g_idx, bits) for q in (q1, q2, q3)]
    assert torch.equal(w, torch.cat(parts, dim=1))
    assert torch.equal(f.bias, torch.cat([q1.bias, q2.bias, q3.bias]))


def test_concat_refuses_layers_that_cannot_share_a_product():
    q1, L1 = member(1, 256, 64, 4, 64)
    q2, _ = member(2, 256, 64, 4, 64)                       # its own activation order
    with pytest.raises(ValueError):
        fused.concat_qlinears([q1, q2])
    q3, _ = member(3, 256, 64, 3, 64, g_idx=L1["g_idx"])    # other width
    with pytest.raises(ValueError):
        fused.concat_qlinears([q1, q3])
    q4, _ = member(4, 256, 64, 4, 64, g_idx=L1["g_idx"], bias=False)
    with pytest.raises(ValueError):
        fused.concat_qlinears([q1, q4])


class Counting(torch.nn.Module):
    infeatures = 8

    def __init__(self):
        super().__init__()
        self.calls = 0

    def forward(self, x):
        self.calls += 1
        return torch.cat([x, 2 * x, 3 * x], dim=-1)


def test_members_share_one_product_per_input_tensor():
    prod = Counting()
    shared = fused.SharedProduct(prod, ("q", "k", "v"))
    q, k, v = (fused.FusedMember(shared, n, 8 * i, 8) for i, n in enumerate(("q", "k", "v")))
    x = torch.randn(2, 8)
    assert torch.equal(q(x), x) and torch.equal(k(x), 2 * x) and torch.equal(v(x), 3 * x)
    assert prod.calls == 1 and shared._x is None           # everyone served: nothing kept alive
    y = torch.randn(2, 8)
    assert torch.equal(k(y), 2 * y) and prod.calls == 2     # any member may come first
    assert torch.equal(k(y), 2 * y) and prod.calls == 3     # the same member again: a new product
    assert torch.equal(q(y), y) and prod.calls == 3
    y.add_(1.0)                                             # modified in place: not the same input
    assert torch.equal(v(y), 3 * y) and prod.calls == 4
    z = y.clone()                                           # equal values, another tensor
    assert torch.equal(q(z), z) and prod.calls == 5


def test_fuse_shared_input_layers_rewrites_the_blocks(tmp_path):
    from autogptq.tvm_amd.loader import from_quantized

    build_checkpoint(str(tmp_path), bits=4, gs=32, act_order=True, shared_order=True)
    model, _ = from_quantized(str(tmp_path), device="cpu")
    names = fused.fuse_shared_input_layers(model)
    assert len(names) == 4 and "model.layers.0.self_attn.q_proj+k_proj+v_proj" in names
    attn = model.model.layers[0].self_attn
    assert isinstance(attn.q_proj, fused.FusedMember) and attn.k_proj.start == 64 and attn.v_proj.start == 128
    assert attn.fused_q_proj_k_proj_v_proj.fused.outfeatures == 192
    assert isinstance(attn.o_proj, QuantLinear)
    mlp = model.model.layers[1].mlp
    assert mlp.fused_gate_proj_up_proj.fused.outfeatures == 256 and isinstance(mlp.down_proj, QuantLinear)
    # the fused weights are listed once
    keys = [k for k in model.state_dict() if "layers.0.self_attn" in k and k.endswith("qweight")]
    assert sorted(keys) == ["model.layers.0.self_attn.fused_q_proj_k_proj_v_proj.fused.qweight",
                            "model.layers.0.self_attn.o_proj.qweight"]


def test_layers_with_their_own_order_stay_separate(tmp_path):
    from autogptq.tvm_amd.loader import from_quantized

    build_checkpoint(str(tmp_path), bits=4, gs=32, act_order=True, shared_order=False)
    model, _ = from_quantized(str(tmp_path), device="cpu")
    assert fused.fuse_shared_input_layers(model) == []
    assert isinstance(model.model.layers[0].self_attn.q_proj, QuantLinear)


@pytest.mark.gpu
@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("M", [1, 5])
def test_fused_members_match_the_separate_layers(bits, M):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    dev = torch.device("cuda:0")
    K, gs = 1024, 128
    q1, L1 = member(11, K, 256, bits, gs)
    q2, _ = member(12, K, 512, bits, gs, g_idx=L1["g_idx"])
    q3, _ = member(13, K, 128, bits, gs, g_idx=L1["g_idx"])
    holder = torch.nn.Module()
    holder.q_proj, holder.k_proj, holder.v_proj = q1.to(dev), q2.to(dev), q3.to(dev)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(3)).half().to(dev)
    want = [l(x).float().cpu() for l in (holder.q_proj, holder.k_proj, holder.v_proj)]
    assert fused.fuse_group(holder, ("q_proj", "k_proj", "v_proj")) is not None
    got = [l(x).float().cpu() for l in (holder.q_proj, holder.k_proj, holder.v_proj)]
    for g, w in zip(got, want):
        assert g.shape == w.shape
        assert float((g - w).abs().max()) <= 3e-3 + 2e-3 * float(w.abs().max())


@pytest.mark.gpu
def test_fused_model_matches_the_unfused_one(tmp_path):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from autogptq.tvm_amd.loader import from_quantized

    cfg, _, _ = build_checkpoint(str(tmp_path), bits=4, gs=32, act_order=True, seed=4, shared_order=True)
    plain, _ = from_quantized(str(tmp_path), device="cuda:0", keep_checkpoint_tensors=True)
    merged, _ = from_quantized(str(tmp_path), device="cuda:0", fuse_shared_inputs=True, prepare_decode=True)
    assert isinstance(merged.model.layers[0].self_attn.k_proj, fused.FusedMember)
    assert merged.model.layers[0].mlp.down_proj._sorted is not None       # prepared at load
    ids = torch.randint(0, cfg.vocab_size, (2, 9), generator=torch.Generator().manual_seed(5)).to("cuda:0")
    with torch.no_grad():
        a = plain(ids).logits.float().cpu()
        b = merged(ids).logits.float().cpu()
        b1 = merged(ids[:, :1]).logits.float().cpu()      # one token per sequence: the decode kernels
        a1 = plain(ids[:, :1]).logits.float().cpu()
    assert np.isfinite(b.numpy()).all()
    assert float((a - b).abs().max()) <= 1e-2 + 1e-2 * float(a.abs().max())
    assert float((a1 - b1).abs().max()) <= 1e-2 + 1e-2 * float(a1.abs().max())


@pytest.mark.gpu
@pytest.mark.parametrize("fuse", [False, True])
def test_compact_model_matches_the_plain_one(tmp_path, fuse):
    """from_quantized as it loads by default: every layer keeps the tiled copy as its only weights (checkpoint
    tensors released, fused projections included) and the model gives the same logits for a prompt and for one
    token as the one that kept the checkpoint tensors."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from autogptq.tvm_amd.loader import from_quantized

    cfg, _, _ = build_checkpoint(str(tmp_path), bits=4, gs=32, act_order=True, seed=6, shared_order=True)
    plain, _ = from_quantized(str(tmp_path), device="cuda:0", keep_checkpoint_tensors=True)
    assert not any(m._compact for m in plain.modules() if isinstance(m, QuantLinear))
    compact, _ = from_quantized(str(tmp_path), device="cuda:0", fuse_shared_inputs=fuse)
    quant = [m for m in compact.modules() if isinstance(m, QuantLinear)]
    assert quant and all(m._compact and m.qweight.numel() == 0 and m.route(1) == "tiled" for m in quant)
    ids = torch.randint(0, cfg.vocab_size, (2, 9), generator=torch.Generator().manual_seed(7)).to("cuda:0")
    for part in (ids, ids[:, :1]):
        with torch.no_grad():
            a = plain(part).logits.float().cpu()
            b = compact(part).logits.float().cpu()
        assert np.isfinite(b.numpy()).all()
        assert float((a - b).abs().max()) <= 1e-2 + 1e-2 * float(a.abs().max())
