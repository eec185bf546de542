"""Drop-in for MoE-Quant's pack_quantized_model.py: pack_weight (the compressed_tensors "pack-quantized" int32
layout, packed by the HIP kernel), the quantization_config it writes, the per-block step that swaps quantized
linears into a block's state dict and saves one safetensors shard, and the command line that walks a whole
checkpoint (`python -m moe_quant_amd.pack_quantized_model --model_name_or_path ... --quantized_model_path ...
--packed_model_path ...`, the reference's arguments).  The command line reads the checkpoint's own
`model.safetensors.index.json` instead of the reference's hard-coded 163 DeepSeek shards and edits `config.json`
as JSON instead of going through transformers' remote-code config class; the files it writes are the same."""
from __future__ import annotations

import argparse
import json
import os
import re
import shutil
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


def prepare_quantization_config(bits, group_size: Optional[int] = None, quantize_only_experts: Optional[bool] = None) -> Dict[str, Any]:
    """pack_quantized_model.py:78-109.  Called as the reference calls it, with one namespace that carries `bits`,
    `group_size` and `quantize_only_experts` (the reference's `args`), or with the three values."""
    if group_size is None and quantize_only_experts is None and hasattr(bits, "bits"):
        args = bits
        bits, group_size, quantize_only_experts = args.bits, args.group_size, args.quantize_only_experts
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


# ---- the whole checkpoint (pack_quantized_model.py:112-243) -------------------------------------------------
class _Shards:
    """Tensors of a sharded safetensors checkpoint by name; shard files are opened on demand."""

    def __init__(self, weight_dir: str):
        self.dir = weight_dir
        idx = os.path.join(weight_dir, "model.safetensors.index.json")
        if os.path.exists(idx):
            with open(idx) as f:
                self.weight_map = dict(json.load(f)["weight_map"])
        else:  # a single file
            from safetensors import safe_open

            with safe_open(os.path.join(weight_dir, "model.safetensors"), framework="pt", device="cpu") as f:
                self.weight_map = {k: "model.safetensors" for k in f.keys()}

    def load(self, keys: Iterable[str]) -> Dict[str, torch.Tensor]:
        from safetensors import safe_open

        by_file = defaultdict(list)
        for k in keys:
            by_file[self.weight_map[k]].append(k)
        out = {}
        for fn, ks in by_file.items():
            with safe_open(os.path.join(self.dir, fn), framework="pt", device="cpu") as f:
                for k in ks:
                    out[k] = f.get_tensor(k)
        return out


def pack_checkpoint(model_name_or_path: str, quantized_model_path: str, packed_model_path: str,
                    dtype: torch.dtype = torch.float16) -> Dict[str, str]:
    """pack_quantized_model.py:112-243 for any checkpoint with `model.layers.<i>.` blocks: shard 1 holds the
    embeddings, one shard per block follows (FP8 tensors dequantized to `dtype`, quantized linears replaced by
    weight_packed / weight_shape / weight_scale), the last shard holds what is left (lm_head, final norm).
    Writes the weight map, `config.json` with the compressed-tensors `quantization_config`, and copies tokenizer,
    generation config and modeling scripts when the source directory has them.  Returns the weight map."""
    from . import quant_utils

    meta = torch.load(os.path.join(quantized_model_path, "metadata.pt"), weights_only=True)
    bits, group_size, only_experts = int(meta["bits"]), int(meta["group_size"]), bool(meta["quantize_only_experts"])
    sym = True  # asymmetric quantization is not supported (pack_quantized_model.py:137-138)
    shards = _Shards(model_name_or_path)
    block_keys = defaultdict(list)
    rest = []
    for k in shards.weight_map:
        m = re.match(r"model\.layers\.(\d+)\.", k)
        (block_keys[int(m.group(1))] if m else rest).append(k)
    n_blocks = max(block_keys) + 1 if block_keys else 0
    cfg_path = os.path.join(model_name_or_path, "config.json")
    cfg = {}
    if os.path.exists(cfg_path):
        with open(cfg_path) as f:
            cfg = json.load(f)
    # The reference walks the blocks of the model built from config.json (pack_quantized_model.py:140-186): tensors
    # of layers beyond num_hidden_layers (DeepSeek-V3's multi-token-prediction layer 61) belong to no block of that
    # model and are not written.
    if isinstance(cfg.get("num_hidden_layers"), int):
        n_blocks = min(n_blocks, cfg["num_hidden_layers"])
    num_output_shards = n_blocks + 2
    quantized = quantized_layers_by_block(quantized_model_path)
    index: Dict[str, str] = {}
    os.makedirs(packed_model_path, exist_ok=True)
    first = [k for k in rest if k == "model.embed_tokens.weight"]
    save_packed_shard(shards.load(first), packed_model_path, 1, num_output_shards, index)
    def dequantized(sd):  # FP8 weights visit the GPU: one fused pass there instead of the padded torch path
        for k, v in list(sd.items()):
            if v.dtype == torch.float8_e4m3fn and torch.cuda.is_available():
                sd[k] = v.cuda()
        quant_utils.dequantize_state_dict(sd, dtype)
        return {k: v.cpu() for k, v in sd.items()}

    for b in range(n_blocks):
        sd = dequantized(shards.load(block_keys[b]))
        sd = pack_block_state_dict(sd, quantized_model_path, quantized.get(b, []), bits, sym, group_size)
        save_packed_shard(sd, packed_model_path, b + 2, num_output_shards, index)
        del sd
    last = [k for k in rest if k not in first]
    save_packed_shard(dequantized(shards.load(last)), packed_model_path, num_output_shards, num_output_shards, index)
    save_safetensors_index(packed_model_path, index)
    cfg.pop("quantization_config", None)  # the source's FP8 description no longer applies (pack_quantized_model.py:118-119)
    cfg["quantization_config"] = prepare_quantization_config(bits, group_size, only_experts)
    with open(os.path.join(packed_model_path, "config.json"), "w") as f:
        json.dump(cfg, f, indent=2)
    for fn in sorted(os.listdir(model_name_or_path)):
        if fn == "config.json" or fn.endswith(".safetensors") or fn == "model.safetensors.index.json":
            continue
        if fn.endswith((".py", ".model", ".txt")) or fn.startswith(("tokenizer", "special_tokens", "generation_config", "vocab",
                                                                     "merges", "added_tokens")):
            src = os.path.join(model_name_or_path, fn)
            if os.path.isfile(src):
                shutil.copy(src, packed_model_path)
    return index


def parse_args(argv=None) -> argparse.Namespace:
    """pack_quantized_model.py:18-49."""
    parser = argparse.ArgumentParser()
    parser.add_argument("--model_name_or_path", type=str, required=True, help="Path to the original checkpoint directory")
    parser.add_argument("--quantized_model_path", type=str, required=True, help="Path to quantized model.")
    parser.add_argument("--packed_model_path", type=str, required=True, help="Where to save the packed model.")
    parser.add_argument("--dtype", default="float16", type=str, choices=["float16", "bfloat16"], help="Torch dtype used.")
    return parser.parse_args(argv)


def main(argv=None) -> None:
    args = parse_args(argv)
    pack_checkpoint(args.model_name_or_path, args.quantized_model_path, args.packed_model_path, getattr(torch, args.dtype))


if __name__ == "__main__":
    main()
