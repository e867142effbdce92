"""MI355X-native GPTQ int3/int4 ``QuantLinear``: the fp16 x packed-weight product behind
``QuantLinear.forward``, on hand-written HIP kernels reached through a C ABI."""
from .qlinear import QuantLinear  # noqa: F401
from . import loader, ops, pack  # noqa: F401
from .loader import find_layers, from_quantized, make_quant  # noqa: F401

__all__ = ["QuantLinear", "ops", "pack", "loader", "find_layers", "make_quant", "from_quantized"]
