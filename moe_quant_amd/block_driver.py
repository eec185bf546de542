"""Per-block calibration driver: the body of MoE-Quant's block loop (quant.py:241-411) on one GPU.

Given one transformer block already on the device and its calibration inputs it
  1. creates a GPTQ handle per nn.Linear (up_proj tied to its gate_proj when asked, quant.py:258-277),
  2. collects the Hessians through forward hooks while the block runs on the calibration inputs (:279-284),
  3. quantizes the shared linears, then the routed experts (:291-386), replaces every weight by its dequantized
     value and writes `<save_dir>/<layer_name>/quantized_weight.pt` = {"qweight", "scale", "zero"} (:323-326),
  4. reports the three issue counters (:332-337, :398-403).
`save_metadata` writes `<save_dir>/metadata.pt` (:428-435); `get_resume_block_idx` is :91-97.

What differs from the reference, on purpose: linears of one shape (the experts) are quantized `group` at a time
through grouped library calls, the groups are queued round-robin on HIP streams, and nothing is read back while
they are queued (the finite check, the issue flags and the files come after one synchronisation);
handles are released without `torch.cuda.empty_cache()`.  Model loading, dataset handling, the distributed
expert split and wandb logging are not part of this engine."""
from __future__ import annotations

import os
import re
from dataclasses import dataclass, field
from typing import Callable, Dict, Iterable, List, Optional

import torch
import torch.nn as nn

from . import quant_utils
from .gptq import GPTQ

ROUTED_EXPERTS_REGEX = r".*mlp.experts.\d+.(down|gate|up)_proj$"  # quant.py:22
LINEAR_LAYERS = (nn.Linear,)  # src/model_utils.py:8


def select_layers(model: nn.Module, layer_prefix: str = "", layer_regex: str = ".*", layer_classes=nn.Module) -> Dict[str, nn.Module]:
    """src/model_utils.py:15-30."""
    layers = {}
    for layer_name, layer in model.named_modules():
        if isinstance(layer, layer_classes) and re.search(layer_regex, layer_name) and layer_name.startswith(layer_prefix):
            layers[layer_name] = layer
    return layers


def get_resume_block_idx(save_dir) -> int:
    """quant.py:91-97: the largest block index that already has a directory under save_dir."""
    resume_block_idx = 0
    if os.path.exists(save_dir):
        for layer_name in os.listdir(save_dir):
            parts = layer_name.split(".")
            if len(parts) > 2 and parts[2].isdigit():
                resume_block_idx = max(resume_block_idx, int(parts[2]))
    return resume_block_idx


def save_metadata(save_dir, bits: int, group_size: int, quantize_only_experts: bool) -> None:
    """quant.py:428-435."""
    os.makedirs(save_dir, exist_ok=True)
    torch.save({"bits": bits, "group_size": group_size, "quantize_only_experts": quantize_only_experts},
               os.path.join(save_dir, "metadata.pt"))


@dataclass
class BlockReport:
    shared: Dict[str, int] = field(default_factory=lambda: {"zero_samples": 0, "nan_hessian": 0, "non_invertible": 0})
    experts: Dict[str, int] = field(default_factory=lambda: {"zero_samples": 0, "nan_hessian": 0, "non_invertible": 0})
    tokens_collected: Dict[str, int] = field(default_factory=dict)
    relative_error: Dict[str, float] = field(default_factory=dict)  # filled with log_error=True
    layers: List[str] = field(default_factory=list)


@torch.no_grad()
def quantize_block(
    model: nn.Module,
    prefix: str,
    run_block: Callable[[], None],
    *,
    bits: int = 4,
    group_size: Optional[int] = 128,
    sym: bool = True,
    rel_damp: float = 1e-2,
    block_size: int = 128,
    quantization_order: str = "default",
    quantization_scale: str = "absmax",
    quantize_only_experts: bool = False,
    tie_gptq_handles: bool = False,
    save_dir: Optional[str] = None,
    log_error: bool = False,
    streams: int = 2,
    group: int = 8,
) -> BlockReport:
    """`model`: any module whose linears under `prefix` are to be quantized (names as in `named_modules()`).
    `run_block()`: runs the block once over every calibration sequence (what quant.py:280-281 does); the forward
    hooks installed here see the inputs of every linear (bf16, fp16 or fp32 activations)."""
    layers = select_layers(model, prefix, ".*", LINEAR_LAYERS)
    handles: Dict[str, GPTQ] = {}
    hooks = {}

    def update_handle_hook(name):
        def _hook(_, inp, out):
            handles[name].update(inp[0])

        return _hook

    for layer_name, layer in layers.items():
        if quantize_only_experts and re.search(ROUTED_EXPERTS_REGEX, layer_name) is None:
            continue
        tied = None
        if tie_gptq_handles and layer_name.endswith("up_proj"):
            parent_name, _ = layer_name.rsplit(".", 1)
            tied = handles[f"{parent_name}.gate_proj"]
        handles[layer_name] = GPTQ(layer, group_size, sym, rel_damp, block_size, quantization_order, quantization_scale,
                                   is_distributed=False, tied_gptq_handle=tied)
        if tied is None:
            hooks[layer_name] = layer.register_forward_hook(update_handle_hook(layer_name))

    run_block()  # collect Hessians
    for h in hooks.values():
        h.remove()

    shared = {k: v for k, v in handles.items() if re.search(ROUTED_EXPERTS_REGEX, k) is None}
    experts = {k: v for k, v in handles.items() if k not in shared}
    report = BlockReport(layers=list(handles))
    dev = next(iter(layers.values())).weight.device if layers else torch.device("cuda")
    main = torch.cuda.current_stream(dev)
    lanes = [main] + [torch.cuda.Stream(device=dev) for _ in range(max(1, streams) - 1)]

    group_size_ = group

    def run_group(group: Dict[str, GPTQ], counters: Dict[str, int]) -> None:
        for ln in lanes:
            if ln is not main:
                ln.wait_stream(main)
        results = {}
        # a tied up_proj must follow its gate_proj on the same stream: units of work are (gate, up) pairs
        units: List[List[str]] = []
        unit_of = {}
        for name in group:  # owners first, in registration order
            if group[name].tied_gptq_handle is None:
                unit_of[id(group[name])] = len(units)
                units.append([name])
        for name in group:
            t = group[name].tied_gptq_handle
            if t is not None:
                if id(t) in unit_of:
                    units[unit_of[id(t)]].append(name)
                else:  # its owner belongs to the other group and is finished already
                    units.append([name])
        # units of one shape and configuration share grouped library calls, `group` units at a time
        buckets: Dict[tuple, List[List[str]]] = {}
        for unit in units:
            h = group[unit[0]]
            buckets.setdefault((h.d_row, h.d_col, h.W_dtype, h.W_device), []).append(unit)
        batches = [b[i:i + max(1, group_size_)] for b in buckets.values() for i in range(0, len(b), max(1, group_size_))]
        for i, batch in enumerate(batches):
            lane = lanes[i % len(lanes)]
            with torch.cuda.stream(lane):
                names = [name for unit in batch for name in unit]
                outs = GPTQ.quantize_many([group[n] for n in names], bits)
                for name, (qweight, scale, zero) in zip(names, outs):
                    h = group[name]
                    deq = quant_utils.dequantize_linear_weight(qweight, scale, zero)
                    err = None
                    if log_error:
                        err = quant_utils.get_relative_mse_error(deq.float(), h.layer.weight.float(), h.H)
                    results[name] = (qweight, scale, zero, deq, torch.isfinite(deq).all(), err)
                    h.layer.weight.data = deq  # quant.py:328
                for name in names:  # release the handle's state (reset() without emptying the allocator cache)
                    h = group[name]
                    h.H = None
                    h._hessian_inv = h._loop_factor = None
                    h._Qt = None
                    h.W = h.layer.weight
        for ln in lanes:
            if ln is not main:
                main.wait_stream(ln)
        torch.cuda.synchronize(dev)
        for name, (qweight, scale, zero, deq, finite, err) in results.items():
            h = group[name]
            assert finite.item(), f"{name} weight is broken after quantization."  # quant.py:299-301
            counters["zero_samples"] += int(h.issue_zero_samples)
            counters["nan_hessian"] += int(h.issue_nan_hessian)
            counters["non_invertible"] += int(h.issue_non_invertible)
            owner = h.tied_gptq_handle if h.tied_gptq_handle is not None else h
            report.tokens_collected[name] = owner.tokens_collected
            if err is not None and not h.has_hessian_issues():
                report.relative_error[name] = float(err.item())
            if save_dir:
                os.makedirs(os.path.join(save_dir, name), exist_ok=True)
                torch.save({"qweight": qweight, "scale": scale, "zero": zero},
                           os.path.join(save_dir, name, "quantized_weight.pt"))

    run_group(shared, report.shared)  # shared handles first (quant.py:291)
    run_group(experts, report.experts)
    return report
