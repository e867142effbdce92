"""Layers that read the same input as one product over their concatenated output columns.

In a decoder block q/k/v projections share one input, and so do gate/up (the reference lists them
as groups that are quantised from the same inputs, auto_gptq/modeling/llama.py:8-12); because the
activation order of GPTQ depends on the inputs only, such layers also share ``g_idx``.  At decode
sizes every product is a launch of a few microseconds that cannot fill the GPU with 4096 output
columns, so three launches over [K, 4096] cost about three times one launch over [K, 12288].
``fuse_shared_input_layers`` concatenates ``qweight`` / ``qzeros`` / ``scales`` / ``bias`` of such
a group along N into one ``QuantLinear`` and replaces the members by views that return their
slice of its output: the model code above (which calls ``q_proj(x)``, ``k_proj(x)``, ``v_proj(x)``
one after the other) needs no change.
"""
from __future__ import annotations

from typing import Dict, Iterable, List, Optional, Sequence

import torch
import torch.nn as nn

from .qlinear import QuantLinear

# groups of layers that read the same tensor, by the names transformers' Llama-like blocks use
# (auto_gptq/modeling/llama.py:8-12 lists the same groups for quantisation)
SHARED_INPUT_GROUPS = (("q_proj", "k_proj", "v_proj"), ("gate_proj", "up_proj"))


def concat_qlinears(layers: Sequence[QuantLinear]) -> QuantLinear:
    """One ``QuantLinear`` whose output is the concatenation of the outputs of ``layers``.  They must
    agree in bits, group size, input width, ``g_idx`` and in having a bias or not."""
    first = layers[0]
    for l in layers[1:]:
        if (l.bits, l.groupsize, l.infeatures) != (first.bits, first.groupsize, first.infeatures):
            raise ValueError("layers differ in bits, group size or input width")
        if (l.bias is None) != (first.bias is None):
            raise ValueError("either every layer has a bias or none")
        if l.g_idx.device != first.g_idx.device or not torch.equal(l.g_idx, first.g_idx):
            raise ValueError("layers differ in g_idx: they were not quantised from the same input")
    out = sum(l.outfeatures for l in layers)
    fused = QuantLinear(first.bits, first.groupsize, first.infeatures, out, first.bias is not None,
                        kernel_switch_threshold=first.kernel_switch_threshold,
                        sort_for_decode=first.sort_for_decode, tile_for_prefill=first.tile_for_prefill)
    fused.qweight = torch.cat([l.qweight for l in layers], dim=1).contiguous()
    fused.qzeros = torch.cat([l.qzeros for l in layers], dim=1).contiguous()    # 32 columns per `bits` words
    fused.scales = torch.cat([l.scales for l in layers], dim=1).contiguous()
    fused.g_idx = first.g_idx.clone()
    if first.bias is not None:
        fused.bias = torch.cat([l.bias for l in layers]).contiguous()
    return fused


class SharedProduct(nn.Module):
    """Holds the fused layer of one group and the result of its last product while members still have
    to pick their slice up."""

    def __init__(self, fused: QuantLinear, names: Sequence[str]):
        super().__init__()
        self.fused = fused
        self.names = tuple(names)
        self._x = None        # the input tensor object the cached product belongs to
        self._version = -1
        self._y = None
        self._pending = set()

    def result_for(self, name: str, x: torch.Tensor) -> torch.Tensor:
        # A hit needs the very same tensor object, unmodified, and a member that has not been served
        # from this product yet; the cache keeps x alive, so the identity cannot be a reused address.
        if not (self._y is not None and x is self._x and x._version == self._version and name in self._pending):
            self._y = self.fused(x)
            self._x, self._version = x, x._version
            self._pending = set(self.names)
        self._pending.discard(name)
        y = self._y
        if not self._pending:   # everyone served: drop the references
            self._x = self._y = None
        return y


class FusedMember(nn.Module):
    """Stands where one layer of a fused group stood: ``forward(x)`` returns that layer's columns of
    the group's product (computed once per input tensor)."""

    def __init__(self, shared: SharedProduct, name: str, start: int, width: int):
        super().__init__()
        # not registered as a submodule: the fused weights are listed once, under the group's owner
        object.__setattr__(self, "_shared", shared)
        self.member_name = name
        self.start = start
        self.outfeatures = width
        self.infeatures = shared.fused.infeatures

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        y = self._shared.result_for(self.member_name, x)
        return y[..., self.start:self.start + self.outfeatures]

    def extra_repr(self) -> str:
        return f"{self.member_name}: columns {self.start}..{self.start + self.outfeatures} of a fused product"


def fuse_group(parent: nn.Module, names: Sequence[str], attr: Optional[str] = None) -> Optional[SharedProduct]:
    """Fuses the children ``names`` of ``parent`` if all are ``QuantLinear`` layers that can share a
    product; returns the ``SharedProduct`` (registered on ``parent`` as ``attr``) or None."""
    members = [getattr(parent, n, None) for n in names]
    if not all(isinstance(m, QuantLinear) for m in members):
        return None
    if any(m.qweight.device.type == "meta" for m in members):
        return None
    try:
        fused = concat_qlinears(members)
    except ValueError:
        return None
    shared = SharedProduct(fused, names)
    start = 0
    for n, m in zip(names, members):
        setattr(parent, n, FusedMember(shared, n, start, m.outfeatures))
        start += m.outfeatures
    setattr(parent, attr or ("fused_" + "_".join(names)), shared)
    return shared


def fuse_shared_input_layers(model: nn.Module, groups: Iterable[Sequence[str]] = SHARED_INPUT_GROUPS) -> List[str]:
    """Fuses, in place, every group of sibling ``QuantLinear`` layers named in ``groups`` below
    ``model``.  The members' own tensors are released (their state-dict entries move under the fused
    layer's name), so this is for inference after loading.  Returns the qualified names of the fused
    groups."""
    done = []
    for mod_name, mod in list(model.named_modules()):
        for names in groups:
            if fuse_group(mod, names) is not None:
                done.append((mod_name + "." if mod_name else "") + "+".join(names))
    return done


__all__ = ["SHARED_INPUT_GROUPS", "concat_qlinears", "fuse_group", "fuse_shared_input_layers", "FusedMember",
           "SharedProduct"]
