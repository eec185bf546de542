"""moe_quant_amd: MI355X-native GPTQ engine behind MoE-Quant's Python API.

Module names mirror the reference's `src` package, so `from moe_quant_amd import gptq, gptq_loop,
linalg_utils, quant_utils` replaces `from src import ...`, and `moe_quant_amd.pack_quantized_model.pack_weight`
replaces the function of the same name in the reference's packing script."""
from . import gptq, gptq_loop, linalg_utils, pack_quantized_model, quant_utils  # noqa: F401
from .gptq import GPTQ  # noqa: F401

__all__ = ["GPTQ", "gptq", "gptq_loop", "linalg_utils", "quant_utils", "pack_quantized_model"]
