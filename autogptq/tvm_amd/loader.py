"""Loading a standard AutoGPTQ checkpoint onto the MI355X ``QuantLinear``.

Mirrors the pieces of the reference's loading path that touch the quantised layers:

* ``find_layers``   auto_gptq/modeling/_utils.py:38-49
* ``make_quant``    auto_gptq/modeling/_utils.py:59-90 (the ``use_tvm=True`` branch picks this
                    package's ``QuantLinear`` instead of ``qlinear_tvm.QuantLinear``)
* ``pack_model``    auto_gptq/modeling/_utils.py:123-157: the layers a GPTQ run quantised, packed in place
* ``save_quantized`` auto_gptq/modeling/_base.py:381-401: the checkpoint directory ``from_quantized`` reads
* ``from_quantized`` auto_gptq/modeling/_base.py:478-569: read ``quantize_config.json``, build the
  model from its config with empty weights, swap the linear layers, load the checkpoint tensors
  by name onto the device.

The checkpoint is read with ``safetensors`` or ``torch.load(weights_only=True)``: nothing from the
file is executed.  Unlike the reference's TVM module, ``QuantLinear`` here can be built on the
``meta`` device (its constructor compiles and allocates nothing on the GPU).
"""
import json
import os
from typing import Dict, Iterable, Optional

import torch
import torch.nn as nn

from .qlinear import QuantLinear


def _conv1d_type():
    try:
        from transformers.pytorch_utils import Conv1D

        return Conv1D
    except Exception:  # transformers missing or too old: no Conv1D layers to find
        return None


def find_layers(module: nn.Module, layers=None, name: str = "") -> Dict[str, nn.Module]:
    """``{qualified name: layer}`` of every Linear / Conv2d / Conv1D in ``module`` (``module`` itself under
    ``name`` when it is one); ``layers`` names other layer types to look for.  Same result as the reference's
    helper (auto_gptq/modeling/_utils.py:38-49), including its order (depth first, in registration order)."""
    kinds = tuple(layers) if layers else tuple(t for t in (_conv1d_type(), nn.Conv2d, nn.Linear) if t is not None)
    found = {}
    for path, sub in module.named_modules(prefix=name, remove_duplicate=False):
        if isinstance(sub, kinds):
            found[path] = sub
    return found


def make_quant(module: nn.Module, names: Iterable[str], bits: int, groupsize: int, name: str = "") -> None:
    """Replaces, in place, every child whose qualified name is in ``names`` by a ``QuantLinear`` of the
    same shape on the same device (``meta`` included)."""
    if isinstance(module, QuantLinear):
        return
    conv1d = _conv1d_type()
    for child_name, child in list(module.named_children()):
        full = name + "." + child_name if name else child_name
        if full in names and not isinstance(child, QuantLinear):
            if isinstance(child, nn.Linear):
                in_features, out_features = child.in_features, child.out_features
            elif isinstance(child, nn.Conv2d):
                in_features, out_features = child.in_channels, child.out_channels
            elif conv1d is not None and isinstance(child, conv1d):
                in_features, out_features = child.weight.shape[0], child.weight.shape[1]
            else:
                raise TypeError(f"{full}: cannot quantise a {type(child).__name__}")
            device = child.weight.device
            new_layer = QuantLinear(bits, groupsize, in_features, out_features, child.bias is not None)
            setattr(module, child_name, new_layer.to(device))
    for child_name, child in module.named_children():
        make_quant(child, names, bits, groupsize, name + "." + child_name if name else child_name)


def pack_model(model: nn.Module, quantizers: Dict[str, tuple], bits: int, group_size: int) -> Dict[str, QuantLinear]:
    """Turns the layers a GPTQ run has quantised into packed ``QuantLinear`` layers, in place: the counterpart
    of auto_gptq/modeling/_utils.py:123-157 (its ``use_tvm=True`` branch, with this package's module).
    ``quantizers[name] = (quantizer, scale, zero, g_idx)`` as the reference's quantisation loop leaves them
    (``scale`` and ``zero`` of shape [N, G]); the first entry is kept as it is.  Packing runs on the CPU, like
    the reference's; every layer then returns to the device it was on.  Returns ``{name: QuantLinear}``."""
    layers = find_layers(model)
    layers = {n: layers[n] for n in quantizers}
    make_quant(model, quantizers, bits, group_size)
    qlayers = find_layers(model, [QuantLinear])
    packed = {}
    for name, q in qlayers.items():
        if name not in quantizers:
            continue
        _, scale, zero, g_idx = quantizers[name]
        device = q.scales.device
        q.to("cpu")
        q.pack(layers[name].to("cpu"), scale.to("cpu"), zero.to("cpu"), None if g_idx is None else g_idx.to("cpu"))
        q.to(device)
        packed[name] = q
    return packed


def save_quantized(model: nn.Module, save_dir: str, bits: int, group_size: int, desc_act: bool = True,
                   use_safetensors: bool = True, model_basename: Optional[str] = None, damp_percent: float = 0.01,
                   sym: bool = True, true_sequential: bool = True) -> str:
    """Writes a packed model the way the reference lays a checkpoint out (auto_gptq/modeling/_base.py:381-401):
    ``gptq_model-{bits}bit-{group_size}g.{safetensors|bin}`` with every tensor of the state dict under its own
    name, ``quantize_config.json`` with the six fields of the reference's ``BaseQuantizeConfig.to_dict``
    (``_base.py:26-32,54-62``; their defaults are the reference's), and the model's ``config.json`` when it has one.  What
    it writes is what ``from_quantized`` reads.  Layers that kept only their tiled copy (``QuantLinear.compact``)
    have no checkpoint tensors left and cannot be saved.  Returns the path of the weight file."""
    for name, mod in model.named_modules():
        if isinstance(mod, QuantLinear) and getattr(mod, "_compact", False):
            raise ValueError(f"{name} holds only its tiled copy (compact()): the checkpoint tensors are gone; load "
                             f"the model with from_quantized(..., keep_checkpoint_tensors=True) to save it again")
    os.makedirs(save_dir, exist_ok=True)
    if model_basename is None:
        model_basename = f"gptq_model-{bits}bit-{group_size}g"
    state = {k: v.detach().to("cpu").clone().contiguous() for k, v in model.state_dict().items()}
    if use_safetensors:
        from safetensors.torch import save_file

        path = os.path.join(save_dir, model_basename + ".safetensors")
        save_file(state, path)
    else:
        path = os.path.join(save_dir, model_basename + ".bin")
        torch.save(state, path)
    config = getattr(model, "config", None)
    if config is not None and hasattr(config, "save_pretrained"):
        config.save_pretrained(save_dir)
    with open(os.path.join(save_dir, "quantize_config.json"), "w", encoding="utf-8") as f:
        json.dump({"bits": int(bits), "group_size": int(group_size), "damp_percent": float(damp_percent),
                   "desc_act": bool(desc_act), "sym": bool(sym), "true_sequential": bool(true_sequential)}, f, indent=2)
    return path


def read_quantize_config(save_dir: str) -> dict:
    """``quantize_config.json`` as the reference writes it (auto_gptq/modeling/_base.py:66-77)."""
    with open(os.path.join(save_dir, "quantize_config.json"), "r", encoding="utf-8") as f:
        cfg = json.load(f)
    for key in ("bits", "group_size"):
        if key not in cfg:
            raise ValueError(f"quantize_config.json has no '{key}'")
    cfg.setdefault("desc_act", True)
    return cfg


def load_state_dict_file(path: str) -> Dict[str, torch.Tensor]:
    """Tensors of a checkpoint file, read with a loader that executes nothing from the file."""
    if path.endswith(".safetensors"):
        from safetensors.torch import load_file

        return load_file(path, device="cpu")
    return torch.load(path, map_location="cpu", weights_only=True)


def load_quantized_state(model: nn.Module, state: Dict[str, torch.Tensor], device) -> None:
    """Materialises ``model`` (possibly on ``meta``) on ``device`` from ``state``, by name.  Every
    parameter and persistent buffer must be present; the packed tensors keep their integer dtype."""
    device = torch.device(device)
    missing = []
    own = dict(model.named_parameters())
    own.update({k: v for k, v in model.named_buffers()})
    non_persistent = set()
    for mod_name, mod in model.named_modules():
        for b in getattr(mod, "_non_persistent_buffers_set", ()):
            non_persistent.add(mod_name + "." + b if mod_name else b)
    for name, old in own.items():
        if name in non_persistent:
            # not in any checkpoint (e.g. rotary tables): keep the value the constructor computed
            if old.device.type == "meta":
                raise ValueError(f"non-persistent buffer {name} is on the meta device; build the model without "
                                 f"empty buffers")
            owner, _, leaf = name.rpartition(".")
            (model.get_submodule(owner) if owner else model)._buffers[leaf] = old.to(device)
            continue
        if name not in state:
            missing.append(name)
            continue
        new = state[name]
        if tuple(new.shape) != tuple(old.shape):
            raise ValueError(f"{name}: checkpoint shape {tuple(new.shape)} != model shape {tuple(old.shape)}")
        dtype = new.dtype if not old.dtype.is_floating_point else old.dtype
        value = new.to(device=device, dtype=dtype)
        owner, _, leaf = name.rpartition(".")
        mod = model.get_submodule(owner) if owner else model
        if leaf in mod._parameters:
            mod._parameters[leaf] = nn.Parameter(value, requires_grad=False)
        else:
            mod._buffers[leaf] = value
    if missing:
        raise KeyError(f"checkpoint lacks {len(missing)} tensors, e.g. {missing[:4]}")


def from_quantized(save_dir: str, device="cuda:0", model_basename: Optional[str] = None,
                   use_safetensors: bool = True, ignore_layers: Iterable[str] = ("lm_head",),
                   trust_remote_code: bool = False, fuse_shared_inputs: bool = False,
                   prepare_decode: bool = False, prepare_tiled: bool = False, compact: Optional[bool] = None,
                   keep_checkpoint_tensors: bool = False):
    """Builds the ``transformers`` causal LM described by ``save_dir/config.json`` with every linear
    layer (except ``ignore_layers`` prefixes: the reference skips ``lm_head`` and the modules outside
    the decoder stack) replaced by ``QuantLinear``, and fills it from
    ``save_dir/gptq_model-{bits}bit-{group_size}g.{safetensors|bin}``.  ``fuse_shared_inputs`` then merges
    q/k/v and gate/up projections into one product each (``fused.fuse_shared_input_layers``; an inference
    optimisation the reference does not have: the state-dict names of those layers change).
    Every layer the tiled format covers ends up holding ONE copy of its weights, the tiled one
    (``QuantLinear.compact``: the reference's TVM module likewise keeps only its own re-laid weights,
    auto_gptq/nn_modules/qlinear_tvm.py:25-40,105-107): device memory per layer is its packed size, every row count
    runs on the tiled kernels, and no call allocates a copy later.  Such a model cannot be saved again or give
    gradients for its inputs; ``keep_checkpoint_tensors=True`` (or ``compact=False``) keeps the checkpoint's tensors
    instead, and the module then builds the copies it wants on first use: ``prepare_decode`` builds the sorted
    copies of activation-order layers at load instead (needed before capturing such a model in a graph: the
    preparation allocates), ``prepare_tiled`` the copies in the tiled format.
    Returns ``(model, quantize_config)``."""
    import accelerate
    from transformers import AutoConfig, AutoModelForCausalLM

    qcfg = read_quantize_config(save_dir)
    bits, group_size = int(qcfg["bits"]), int(qcfg["group_size"])
    if model_basename is None:
        model_basename = f"gptq_model-{bits}bit-{group_size}g"
    path = os.path.join(save_dir, model_basename + (".safetensors" if use_safetensors else ".bin"))
    if not os.path.isfile(path):
        raise FileNotFoundError(f"Could not find model at {path}")
    config = AutoConfig.from_pretrained(save_dir, trust_remote_code=trust_remote_code)
    with accelerate.init_empty_weights(include_buffers=False):
        model = AutoModelForCausalLM.from_config(config, trust_remote_code=trust_remote_code, torch_dtype=torch.float16)
    layers = find_layers(model)
    for lname in list(layers):
        if any(lname.startswith(prefix) for prefix in ignore_layers):
            del layers[lname]
    with accelerate.init_empty_weights(include_buffers=True):  # the packed buffers too: nothing is allocated
        make_quant(model, layers, bits, group_size)
    state = load_state_dict_file(path)
    # tied output embeddings are stored once
    if hasattr(model, "tie_weights"):
        for tied in ("lm_head.weight",):
            if tied not in state and getattr(config, "tie_word_embeddings", False):
                emb = model.get_input_embeddings()
                for k, v in model.named_parameters():
                    if v is emb.weight and k in state:
                        state[tied] = state[k]
    load_quantized_state(model, state, device)
    if hasattr(model, "tie_weights"):
        model.tie_weights()
    if fuse_shared_inputs:
        from .fused import fuse_shared_input_layers

        fuse_shared_input_layers(model)
    if compact is None:
        compact = not (keep_checkpoint_tensors or prepare_decode or prepare_tiled)
    for mod in model.modules():
        if not isinstance(mod, QuantLinear):
            continue
        if compact and mod.compact():
            continue
        if prepare_decode and mod.sort_for_decode:
            mod.prepare_decode()
        if prepare_tiled and mod.tile_for_prefill:
            mod.prepare_tiled()
    seqlen = 4096
    for key in ("max_position_embeddings", "seq_length", "n_positions"):
        if key in model.config.to_dict():
            seqlen = model.config.to_dict()[key]
            break
    model.seqlen = seqlen
    model.eval()
    return model, qcfg
