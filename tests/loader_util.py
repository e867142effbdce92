"""Builds a tiny quantised Llama checkpoint on disk, the way the reference's save_quantized lays it
out (auto_gptq/modeling/_base.py:428-470): config.json, quantize_config.json,
gptq_model-{bits}bit-{g}g.safetensors with QuantLinear buffers under the original layer names."""
import json
import os

import torch


def rtn_quantize(weight: torch.Tensor, bits: int, gs: int):
    """Round-to-nearest per (column, group): returns scales [N, G], zeros [N, G] as pack() wants them."""
    N, K = weight.shape
    G = K // gs
    w = weight.float().reshape(N, G, gs)
    maxq = (1 << bits) - 1
    lo = torch.minimum(w.min(dim=2).values, torch.zeros(()))
    hi = torch.maximum(w.max(dim=2).values, torch.zeros(()))
    scales = ((hi - lo) / maxq).clamp_min(1e-5)
    zeros = torch.round(-lo / scales).clamp_(1, maxq)
    return scales, zeros


def build_checkpoint(tmp_dir: str, bits: int = 4, gs: int = 32, act_order: bool = True, seed: int = 0,
                     shared_order: bool = False):
    """shared_order: layers that read the same input (q/k/v, gate/up) get the same g_idx, as GPTQ
    produces them (its activation order depends on the inputs only)."""
    from safetensors.torch import save_file
    from transformers import AutoModelForCausalLM, LlamaConfig

    from autogptq.tvm_amd import QuantLinear
    from autogptq.tvm_amd.loader import find_layers

    torch.manual_seed(seed)
    cfg = LlamaConfig(hidden_size=64, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=4, vocab_size=128, max_position_embeddings=64,
                      tie_word_embeddings=False)
    model = AutoModelForCausalLM.from_config(cfg).half()
    state = {k: v.clone() for k, v in model.state_dict().items()}
    dense = {}  # name -> the fp16 weight the quantised layer represents
    gen = torch.Generator().manual_seed(seed + 1)
    shared_g = None
    for name, layer in find_layers(model).items():
        if name.startswith("lm_head"):
            continue
        N, K = layer.weight.shape
        scales, zeros = rtn_quantize(layer.weight.data, bits, gs)
        if act_order:
            g_idx = (torch.randperm(K, generator=gen) // gs).to(torch.int32)
            if shared_order:
                leaf = name.rsplit(".", 1)[-1]
                if leaf in ("k_proj", "v_proj", "up_proj"):
                    g_idx = shared_g
                else:
                    shared_g = g_idx
            # quantise against the permuted grouping so that codes stay in range
            w = layer.weight.data.float()
            G = K // gs
            lo = torch.zeros(N, G)
            hi = torch.zeros(N, G)
            for g in range(G):
                cols = w[:, g_idx == g]
                lo[:, g] = torch.minimum(cols.min(dim=1).values, torch.zeros(()))
                hi[:, g] = torch.maximum(cols.max(dim=1).values, torch.zeros(()))
            maxq = (1 << bits) - 1
            scales = ((hi - lo) / maxq).clamp_min(1e-5)
            zeros = torch.round(-lo / scales).clamp_(1, maxq)
        else:
            g_idx = (torch.arange(K) // gs).to(torch.int32)
        q = QuantLinear(bits, gs, K, N, layer.bias is not None)
        q.pack(layer, scales.clone(), zeros.clone(), g_idx)
        del state[name + ".weight"]
        for buf in ("qweight", "qzeros", "scales", "g_idx"):
            state[f"{name}.{buf}"] = getattr(q, buf).clone().contiguous()
        dense[name] = q
    os.makedirs(tmp_dir, exist_ok=True)
    cfg.save_pretrained(tmp_dir)
    with open(os.path.join(tmp_dir, "quantize_config.json"), "w") as f:
        json.dump({"bits": bits, "group_size": gs, "desc_act": act_order, "damp_percent": 0.01}, f)
    save_file({k: v.contiguous() for k, v in state.items()},
              os.path.join(tmp_dir, f"gptq_model-{bits}bit-{gs}g.safetensors"))
    return cfg, state, dense
