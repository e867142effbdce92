"""MI355X-native GPTQ int3/int4 ``QuantLinear``: the fp16 x packed-weight product behind
``QuantLinear.forward``, on hand-written HIP kernels reached through a C ABI."""
from .qlinear import QuantLinear  # noqa: F401
from . import fused, loader, ops, pack  # noqa: F401
from .fused import fuse_shared_input_layers  # noqa: F401
from .loader import find_layers, from_quantized, make_quant, pack_model, save_quantized  # noqa: F401

__all__ = ["QuantLinear", "ops", "pack", "loader", "fused", "find_layers", "make_quant", "pack_model", "save_quantized", "from_quantized",
           "fuse_shared_input_layers"]
