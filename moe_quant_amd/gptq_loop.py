"""Drop-in for MoE-Quant's src/gptq_loop.py: same call, HIP kernels underneath (no Triton, no graph)."""
from __future__ import annotations

import torch
from torch import Tensor

from . import ops


def gptq_loop(
    weight: Tensor,
    hessian_inv: Tensor,
    scale: Tensor,
    qzero: Tensor,
    maxq: Tensor,
    dtype: torch.dtype,
    gptq_block_size: int = 128,
) -> Tensor:
    """Quantize `weight` with GPTQ (src/gptq_loop.py:193-225).

    weight (C,R) fp32: transposed weights, modified in place to the dequantized values
    hessian_inv (C,C) fp32: unit-diagonal upper factor;  scale, qzero (C,R) fp32;  maxq () fp32
    dtype: rounding dtype of dequantized values (fp16 / bf16 / None)
    Returns qweight (C,R) fp32 holding the integer codes, as the reference does."""
    assert weight.is_contiguous() and hessian_inv.is_contiguous() and scale.is_contiguous() and qzero.is_contiguous()
    if gptq_block_size <= 0:
        gptq_block_size = weight.size(-2)
    Qt = ops.gptq_loop_(weight, hessian_inv, scale, None, qzero, 0.0, float(maxq), dtype, gptq_block_size)
    return Qt.to(weight.dtype)
