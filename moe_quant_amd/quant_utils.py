"""Drop-in for the hot-path part of MoE-Quant's src/quant_utils.py.

get_quantization_grid (absmax, symmetric) runs on the HIP grid kernel; the small elementwise helpers
(quantize / dequantize / round_fp / dequantize_linear_weight / get_relative_mse_error) are the
reference's own torch one-liners and stay torch: they are metrics and test helpers, not the path."""
from __future__ import annotations

import warnings
from enum import Enum
from typing import Optional

import torch
from torch import Tensor

from . import ops


class QuantizationScale(Enum):
    ABSMAX = "absmax"
    MSE = "mse"


def round_fp(x: Tensor, dtype: torch.dtype = None) -> Tensor:
    """src/quant_utils.py:52-53."""
    return x if dtype is None else x.to(dtype=dtype).to(x.dtype)


def quantize(x: Tensor, scale: Tensor, qzero: Tensor, maxq: Tensor) -> Tensor:
    """src/quant_utils.py:57-58 (round-half-even torch helper)."""
    return (x / scale + qzero).round().clamp(torch.zeros_like(maxq), maxq)


def dequantize(qx: Tensor, scale: Tensor, qzero: Tensor, dtype: torch.dtype = None) -> Tensor:
    """src/quant_utils.py:61-62."""
    return round_fp((qx - qzero) * scale, dtype)


def dequantize_quantized(x, scale, qzero, maxq, dtype=None):
    """src/quant_utils.py:65-68."""
    return dequantize(quantize(x, scale, qzero, maxq), scale, qzero, dtype)


def find_quantization_meta(x: Tensor, bit_width: int, symmetric: bool = False, dtype: torch.dtype = None):
    """src/quant_utils.py:75-101 for x of shape (..., G, g): per-group scale, qzero, maxq.  Symmetric only."""
    if not symmetric:
        raise NotImplementedError("only symmetric quantization is supported (as MoE-Quant's README states)")
    *lead, G, g = x.shape
    x2 = x.reshape(-1, G * g)
    scale, _ = ops.quant_grid_sym(x2, g, bit_width, dtype, want_transposed=False)
    maxq = torch.tensor(2**bit_width - 1, dtype=x.dtype, device=x.device)
    scale = scale.to(x.dtype).reshape(*lead, G)
    qzero = torch.full_like(scale, (2**bit_width) * 0.5)
    return scale, qzero, maxq


@torch.no_grad()
def mse_scale(x: Tensor, p: Tensor, scale: Tensor, qzero: Tensor, maxq: Tensor, dtype: torch.dtype = None,
              norm: float = 2.4) -> Tensor:
    """src/quant_utils.py:143-192: x (..., g) weights of each group, p (P,) shrink factors, scale/qzero (...);
    `scale` is modified in place and returned.  Symmetric grids only: one zero point for all groups."""
    assert x.is_contiguous() and p.is_contiguous() and scale.is_contiguous() and qzero.is_contiguous()
    g = x.shape[-1]
    x2 = x.reshape(-1, g)
    z = float(qzero.reshape(-1)[0].item()) if qzero.numel() else 0.0
    sc = scale.reshape(-1, 1).float().contiguous()
    ops.mse_scale_sym_(x2, g, p.float().contiguous(), sc, None, z, float(maxq.item()), norm, dtype)
    scale.copy_(sc.reshape(scale.shape).to(scale.dtype))
    return scale


@torch.no_grad()
def get_quantization_grid(
    weight: Tensor,
    group_size: int,
    bits: int,
    symmetric: bool = False,
    dtype: torch.dtype = None,
    quantization_scale=QuantizationScale.ABSMAX,
    quant_max_shrink: float = 0.2,
    quant_n_grid: int = 100,
    quant_norm: float = 2.4,
):
    """src/quant_utils.py:195-240: returns (scale (...,C), qzero (...,C), maxq ()) replicated per column."""
    # The reference tests `quantization_scale == QuantizationScale.MSE`, which a plain string never satisfies
    # (src/gptq.py:47 stores the string): its search is unreachable from the GPTQ class.  Here both the enum
    # member and the string "mse" select it.
    mse = quantization_scale == QuantizationScale.MSE or quantization_scale == "mse"
    group_size = group_size or weight.shape[-1]
    w = weight.unflatten(dim=-1, sizes=(-1, group_size))
    scale, qzero, maxq = find_quantization_meta(w, bits, symmetric, dtype)
    if mse:
        search_points = torch.linspace(1, quant_max_shrink, quant_n_grid, dtype=torch.float32, device=weight.device)
        scale = mse_scale(w.contiguous(), search_points, scale.contiguous(), qzero, maxq, dtype, quant_norm)
    scale = scale.repeat_interleave(group_size, dim=-1)
    qzero = qzero.repeat_interleave(group_size, dim=-1)
    assert weight.shape == scale.shape == qzero.shape and maxq.shape == ()
    return scale, qzero, maxq


def dequantize_linear_weight(qweight: Tensor, scale: Tensor, zero: Tensor, perm: Optional[Tensor] = None):
    """src/quant_utils.py:243-256."""
    scale = scale.view(qweight.shape[0], -1, 1)
    zero = zero.view(qweight.shape[0], -1, 1)
    num_groups = scale.shape[1]
    weight = dequantize(qweight.view(qweight.shape[0], num_groups, -1), scale, zero).view_as(qweight)
    if perm is not None:
        weight = weight[:, perm.argsort()]
    return weight


def get_relative_mse_error(q: Tensor, w: Tensor, H: Optional[Tensor] = None):
    """src/quant_utils.py:259-264."""
    delta = q - w
    if H is None:
        return delta.pow(2).mean() / w.pow(2).mean()
    return delta.mm(H).mul(delta).mean() / (w.mm(H).mul(w).mean() + 1e-6)


FP8_GROUP_SIZE = 128  # src/quant_utils.py:16
FP8_DTYPES = (torch.float8_e4m3fn, torch.float8_e4m3fnuz, torch.float8_e5m2, torch.float8_e5m2fnuz)  # :17


def dequantize_weight_from_fp8(W: Tensor, s: Tensor) -> Tensor:
    """src/quant_utils.py:267-284.  The reference receives W and s already cast to the target dtype and multiplies
    them block by block.  An FP8 W (with s of the target dtype) takes the fused HIP kernel instead: same values,
    one pass, no padded copies."""
    if W.dtype == torch.float8_e4m3fn:
        if s.dtype not in (torch.bfloat16, torch.float16):
            raise TypeError("with an FP8 weight, s carries the target dtype: cast it to bfloat16 or float16")
        return ops.dequant_fp8_block(W, s, s.dtype)
    if W.dtype in FP8_DTYPES:
        raise NotImplementedError(f"{W.dtype} checkpoints are not supported (DeepSeek ships float8_e4m3fn)")
    g = FP8_GROUP_SIZE
    d_out, d_in = W.shape
    rows = torch.arange(d_out, device=W.device) // g
    cols = torch.arange(d_in, device=W.device) // g
    return W * s[rows][:, cols]


def dequantize_state_dict(state_dict: dict, dtype: torch.dtype = torch.float16) -> None:
    """src/quant_utils.py:287-298: every `<layer>.weight` that has a `<layer>.weight_scale_inv` is replaced by its
    dequantized value in `dtype`, and the scale entry is dropped."""
    for k in list(state_dict.keys()):
        if k.endswith("scale_inv"):
            layer_name, _ = k.rsplit(".", 1)
            W = state_dict[f"{layer_name}.weight"]
            s = state_dict[f"{layer_name}.weight_scale_inv"]
            if W.dtype == torch.float8_e4m3fn and W.is_cuda:
                # the reference rounds the scale to `dtype` first (s.to(dtype)); the kernel does the same
                state_dict[f"{layer_name}.weight"] = ops.dequant_fp8_block(W, s.to(W.device), dtype)
            else:
                state_dict[f"{layer_name}.weight"] = dequantize_weight_from_fp8(W.to(dtype), s.to(dtype))
            del state_dict[f"{layer_name}.weight_scale_inv"]


def can_dequantize_from_fp8(state_dict: dict) -> bool:
    """src/quant_utils.py:301-305."""
    for k, v in state_dict.items():
        if v.dtype in FP8_DTYPES and f"{k}_scale_inv" not in state_dict:
            return False
    return True
