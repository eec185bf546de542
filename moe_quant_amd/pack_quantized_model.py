"""Drop-in for pack_weight of MoE-Quant's pack_quantized_model.py (the compressed_tensors
"pack-quantized" int32 layout), packed by the HIP kernel."""
from __future__ import annotations

from typing import Optional

import torch

from . import ops


def pack_to_int32(value: torch.Tensor, num_bits: int) -> torch.Tensor:
    """compressed_tensors.compressors.pack_to_int32 for num_bits == 4: int8 values in [-8, 7],
    eight per int32 word, element i in bits [4i, 4i+4) after the +8 offset."""
    if value.dtype != torch.int8:
        raise ValueError("Tensor must be quantized to torch.int8 before packing")
    if num_bits > 8:
        raise ValueError("Packing is only supported for less than 8 bits")
    if num_bits != 4:
        raise NotImplementedError("only 4-bit packing is implemented")
    dev = value.device
    v = value if value.is_cuda else value.cuda()
    out = ops.pack_int4((v + 8).to(torch.uint8))
    return out.to(dev)


def pack_weight(weight: dict, bits: int, sym: bool, group_size: Optional[int] = None) -> dict:
    """pack_quantized_model.py:57-75.  Tensors may live on the CPU (as after torch.load in the
    reference's CLI); they are moved to the GPU for packing and the result is returned on their device."""
    if bits != 4:
        raise NotImplementedError("only 4-bit packing is implemented")
    qweight, scale, zero = weight["qweight"], weight["scale"], weight["zero"]
    group_size = group_size or qweight.shape[-1]
    dev = qweight.device
    q = qweight if qweight.is_cuda else qweight.cuda()
    z = zero.to(q.device)
    packed = ops.pack_int4(q.to(torch.uint8), z.float(), group_size)
    out = {
        "weight_packed": packed.to(dev),
        "weight_shape": torch.tensor(qweight.shape),
        "weight_scale": scale,
    }
    if not sym:
        out["weight_zero_point"] = weight["zero"]
    return out
