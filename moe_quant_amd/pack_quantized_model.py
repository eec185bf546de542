"""Drop-in for the model-independent parts of MoE-Quant's pack_quantized_model.py: pack_weight (the
compressed_tensors "pack-quantized" int32 layout, packed by the HIP kernel), the quantization_config it writes,
and the per-block step that swaps quantized linears into a block's state dict and saves one safetensors shard.
Loading the 163-shard DeepSeek checkpoint, the HF config/tokenizer copies and the FP8 dequantization of the
untouched tensors stay with the caller."""
from __future__ import annotations

import json
import os
from collections import defaultdict
from typing import Any, Dict, Iterable, Optional

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


def prepare_quantization_config(bits: int, group_size: int, quantize_only_experts: bool) -> Dict[str, Any]:
    """pack_quantized_model.py:78-109 (takes the three values instead of the argparse namespace)."""
    ignored_modules = ["lm_head"]
    if quantize_only_experts:
        ignored_modules += ["re:.*self_attn.*", "re:.*shared_experts.*", r"re:.*mlp\.(gate|up|gate_up|down)_proj.*"]
    return {
        "config_groups": {
            "group_0": {
                "input_activations": None,
                "output_activations": None,
                "targets": ["Linear"],
                "weights": {
                    "actorder": None,
                    "block_structure": None,
                    "dynamic": False,
                    "group_size": group_size,
                    "num_bits": bits,
                    "observer": "minmax",
                    "observer_kwargs": {},
                    "strategy": "group",
                    "symmetric": True,
                    "type": "int",
                },
            }
        },
        "format": "pack-quantized",
        "ignore": ignored_modules,
        "kv_cache_scheme": None,
        "quant_method": "compressed-tensors",
        "quantization_status": "compressed",
    }


def quantized_layers_by_block(quantized_model_path: str) -> Dict[int, list]:
    """pack_quantized_model.py:143-147: directory names `model.layers.<idx>.<...>` grouped by block index."""
    names = defaultdict(list)
    for layer_name in sorted(os.listdir(quantized_model_path)):
        if os.path.isdir(os.path.join(quantized_model_path, layer_name)):
            names[int(layer_name.split(".")[2])].append(layer_name)
    return names


def pack_block_state_dict(block_state_dict: Dict[str, torch.Tensor], quantized_model_path: str, layer_names: Iterable[str],
                          bits: int, sym: bool, group_size: int) -> Dict[str, torch.Tensor]:
    """pack_quantized_model.py:186-197: for every quantized linear of the block, `<name>.weight` (and the FP8
    `<name>.weight_scale_inv`) leave the state dict and weight_packed / weight_shape / weight_scale enter it."""
    for layer_name in layer_names:
        weight_state_dict = torch.load(os.path.join(quantized_model_path, layer_name, "quantized_weight.pt"),
                                       weights_only=True, map_location="cpu")
        packed = pack_weight(weight_state_dict, bits, sym, group_size)
        block_state_dict.pop(f"{layer_name}.weight")
        block_state_dict.pop(f"{layer_name}.weight_scale_inv", None)
        block_state_dict.update({f"{layer_name}.{k}": v for k, v in packed.items()})
    return block_state_dict


def save_packed_shard(block_state_dict: Dict[str, torch.Tensor], packed_model_path: str, shard_id: int, num_shards: int,
                      safetensors_index: Dict[str, str]) -> str:
    """pack_quantized_model.py:199-206: one safetensors file per block, recorded in the weight map."""
    from safetensors.torch import save_file

    os.makedirs(packed_model_path, exist_ok=True)
    shard = f"model-{shard_id:05}-of-{num_shards:05}.safetensors"
    save_file({k: v.contiguous() for k, v in block_state_dict.items()}, os.path.join(packed_model_path, shard))
    for k in block_state_dict:
        safetensors_index[k] = shard
    return shard


def save_safetensors_index(packed_model_path: str, safetensors_index: Dict[str, str]) -> None:
    """pack_quantized_model.py:232-233."""
    with open(os.path.join(packed_model_path, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": safetensors_index}, f)
