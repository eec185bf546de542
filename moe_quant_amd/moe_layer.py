"""One MoE layer through the engine on one GPU: the expert part of MoE-Quant's per-block flow
(quant.py:241-411) with the model forward replaced by its two ingredients the Hessians need --
the routed token sets and the SwiGLU product that feeds each down projection.

Flow, as in the reference: all Hessians of the block are collected first (gate and up of an expert
share one, quant.py:258-277), then every linear is quantized and packed.  Everything stays resident
in HBM: 256 x 7168^2 fp32 gate/up Hessians (52.6 GB) + 256 x 2048^2 (4.3 GB) + 2M x 7168 bf16 tokens
(30 GB) + bf16 weights (22.5 GB) fit one MI355X.  Routed activations are gathered one expert at a time
(materialising all top-8 copies at once would take 240 GB).
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
import torch.nn as nn

from . import ops
from .gptq import GPTQ


@dataclass
class ExpertWeights:
    gate: torch.Tensor  # (I, C) bf16
    up: torch.Tensor  # (I, C) bf16
    down: torch.Tensor  # (C, I) bf16


@dataclass
class LayerResult:
    seconds: Dict[str, float] = field(default_factory=dict)
    tokens_per_expert: List[int] = field(default_factory=list)
    packed: Dict[str, torch.Tensor] = field(default_factory=dict)  # "<e>.<proj>" -> int32 words (kept if asked)
    scales: Dict[str, torch.Tensor] = field(default_factory=dict)
    qweight: Dict[str, torch.Tensor] = field(default_factory=dict)  # only for the experts listed in keep_codes
    hessians: Dict[str, torch.Tensor] = field(default_factory=dict)  # idem (undamped copies)
    down_inputs: Dict[int, torch.Tensor] = field(default_factory=dict)  # idem: what the expert's down_proj saw
    issues: Dict[str, int] = field(default_factory=dict)
    issues_by_linear: Dict[str, List[str]] = field(default_factory=dict)  # "<e>.<proj>" -> names of raised flags
    factorizations: int = 0  # Hessian factorisations actually computed (a tied up_proj reuses its gate_proj's)
    overlapped: bool = False  # quantization ran beside the collection of later Hessians (seconds then overlap too)


def route_tokens(expert_ids: torch.Tensor, n_experts: int):
    """expert_ids (T, top_k) -> (order, offsets): order[offsets[e]:offsets[e+1]] are the token rows of expert e."""
    flat = expert_ids.reshape(-1)
    order = torch.argsort(flat, stable=True)
    counts = torch.bincount(flat, minlength=n_experts)
    offsets = torch.zeros(n_experts + 1, dtype=torch.int64, device=flat.device)
    offsets[1:] = torch.cumsum(counts, 0)
    return order // expert_ids.shape[1], offsets.tolist()


@torch.no_grad()
def quantize_moe_layer(
    x: torch.Tensor,
    expert_ids: torch.Tensor,
    experts: List[ExpertWeights],
    bits: int = 4,
    group_size: int = 128,
    rel_damp: float = 0.01,
    block_size: int = 128,
    keep_outputs: bool = False,
    keep_codes: Optional[List[int]] = None,
    max_rows_per_update: int = 1 << 17,
    streams: int = 2,
    group: int = 8,
    overlap: bool = True,
) -> LayerResult:
    """x (T, C) bf16 on the GPU, expert_ids (T, top_k) int64 on the GPU.

    `group`, `streams`: one linear is a long chain of dependent launches whose critical path (one-workgroup
    diagonal blocks, 64-row column walks) leaves most of the GPU idle.  Experts are therefore quantized `group` at a
    time -- their factorisations and column loops run as grouped library calls, every launch carrying the work of
    all of them -- and the groups go round-robin onto `streams` HIP streams, so that the short per-linear kernels
    of one group overlap the long launches of another.  Nothing in the path reads a value back to the host, so one
    host thread keeps all streams fed.
    `overlap`: quantize a group as soon as its Hessians are complete, beside the collection of the next group's
    (False: the reference's order, every Hessian of the block first)."""
    dev = x.device
    E = len(experts)
    keep_codes = set(keep_codes or [])
    res = LayerResult()
    sync = lambda: torch.cuda.synchronize(dev)

    def linear(w):
        m = nn.Linear(w.shape[1], w.shape[0], bias=False, dtype=w.dtype, device=dev)
        m.weight.data = w
        return m

    handles = []
    for ew in experts:
        g = GPTQ(linear(ew.gate), group_size, True, rel_damp, block_size)
        u = GPTQ(linear(ew.up), group_size, True, rel_damp, block_size, tied_gptq_handle=g)
        d = GPTQ(linear(ew.down), group_size, True, rel_damp, block_size)
        handles.append((g, u, d))

    sync()
    t0 = time.perf_counter()
    rows, offsets = route_tokens(expert_ids, E)
    sync()
    res.seconds["route"] = time.perf_counter() - t0
    res.tokens_per_expert = [offsets[e + 1] - offsets[e] for e in range(E)]
    main = torch.cuda.current_stream(dev)
    n_lanes = max(1, streams)
    # without overlap the current stream is lane 0; with overlap the Hessians keep the current stream to themselves
    lanes = ([] if overlap else [main]) + [torch.cuda.Stream(device=dev) for _ in range(n_lanes - (0 if overlap else 1))]
    done = []  # (name, handle): verdict words are read after everything is queued
    factor_calls_before = GPTQ.factor_calls
    group = max(1, group)

    # Hessian products wait here until `group` of one width have come together (or the same handle comes again: two
    # products into one H must not share a launch); then they run as one grouped library call.
    pending = {"gate_up": [], "down": []}

    def flush(kind):
        for want_packed in (True, False):
            part = [(h, p) for h, p in pending[kind] if isinstance(p, ops.PackedTokens) == want_packed]
            if part:
                GPTQ.update_many([h for h, _ in part], [p for _, p in part])
        pending[kind].clear()

    def enqueue(kind, h, tokens):
        if any(h is q for q, _ in pending[kind]):
            flush(kind)
        pending[kind].append((h, tokens))
        if len(pending[kind]) >= group:
            flush(kind)

    packable = x.dtype in (torch.bfloat16, torch.float16) and x.shape[1] % 8 == 0 and experts[0].gate.shape[0] % 8 == 0

    def collect_hessians(e):
        """Hessians of expert e (gate and up share one, quant.py:258-277) from its routed tokens: one pass gathers the
        expert's rows of x twice -- token-major for the two GEMMs of the expert's own forward (the model's matmuls,
        rocBLAS/hipBLASLt through torch) and in the packed layout the Hessian kernel reads -- and the SiLU product is
        written straight into that layout, its only reader being the down projection's Hessian."""
        g, u, d = handles[e]
        lo, hi = offsets[e], offsets[e + 1]
        for s in range(lo, hi, max_rows_per_update):
            idx = rows[s : min(hi, s + max_rows_per_update)]
            if packable and idx.numel() >= 256:
                P, xe = ops.pack_tokens(x, idx, also_token_major=True)
                enqueue("gate_up", g, P)
                A = ops.swiglu_packed(xe @ experts[e].gate.t(), xe @ experts[e].up.t())
                enqueue("down", d, A)
                a = ops.unpack_tokens(A) if e in keep_codes else None
            else:  # a handful of tokens: plain tensors
                xe = x.index_select(0, idx)
                enqueue("gate_up", g, xe)
                a = ops.swiglu(torch.cat([xe @ experts[e].gate.t(), xe @ experts[e].up.t()], dim=1))
                enqueue("down", d, a)
            if e in keep_codes:
                prev = res.down_inputs.get(e)
                res.down_inputs[e] = a if prev is None else torch.cat([prev, a])

    def hessians_done():
        flush("gate_up")
        flush("down")

    def quantize_chunk(chunk):
        """Quantize + pack the three linears of every expert of the chunk (on the current stream)."""
        for e in chunk:
            g, u, d = handles[e]
            if e in keep_codes:
                g.symmetrize_hessian()
                d.symmetrize_hessian()
                if g.H is not None:
                    res.hessians[f"{e}.gate_proj"] = g.H.clone()
                if d.H is not None:
                    res.hessians[f"{e}.down_proj"] = d.H.clone()
        # gate and up projections of the chunk (one factor per expert, shared), then the down projections
        gu = [handles[e][i] for e in chunk for i in (0, 1)]
        names = [(e, n) for e in chunk for n in ("gate_proj", "up_proj")] + [(e, "down_proj") for e in chunk]
        dn = [handles[e][2] for e in chunk]
        if group > 1:
            outs = GPTQ.quantize_many(gu, bits) + GPTQ.quantize_many(dn, bits)
        else:
            outs = [h.quantize(bits) for h in gu + dn]
        for (e, name), h, (q, s, z) in zip(names, gu + dn, outs):
            words = h.packed_words()
            done.append((f"{e}.{name}", h))
            if keep_outputs:
                res.packed[f"{e}.{name}"] = words
                res.scales[f"{e}.{name}"] = s
            if e in keep_codes:
                res.qweight[f"{e}.{name}"] = q
                res.scales[f"{e}.{name}"] = s
        for h in gu + dn:  # as quant.py:330: free per-linear state as soon as the linear is done
            h.H = None
            h._hessian_inv = h._loop_factor = None
            h._Qt = None
            h.W = h.layer.weight

    chunks = [list(range(e0, min(E, e0 + group))) for e0 in range(0, E, group)]
    t1 = time.perf_counter()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record(main)
    if overlap:
        # The Hessians of a chunk of experts are collected on the current stream; as soon as they are complete the
        # chunk is quantized on a lane of its own while the next chunk's Hessians are collected.  Legal because the
        # expert forward reads the original weights whatever has been quantized meanwhile (this driver never writes
        # quantized weights back), which is all the reference's "collect everything first" order is there for.
        for ci, chunk in enumerate(chunks):
            for e in chunk:
                collect_hessians(e)
            hessians_done()
            ready = torch.cuda.Event()
            ready.record(main)
            lane = lanes[ci % len(lanes)]
            lane.wait_event(ready)
            with torch.cuda.stream(lane):
                quantize_chunk(chunk)
        ev1.record(main)
    else:
        # ---- phase 1: Hessians of the whole block, phase 2: quantize + pack, chunks round-robin over the lanes
        for chunk in chunks:
            for e in chunk:
                collect_hessians(e)
        hessians_done()
        ev1.record(main)
        sync()
        for s_ in lanes:
            if s_ is not main:
                s_.wait_stream(main)
        for ci, chunk in enumerate(chunks):
            with torch.cuda.stream(lanes[ci % len(lanes)]):
                quantize_chunk(chunk)
    for s_ in lanes:
        if s_ is not main:
            main.wait_stream(s_)
    sync()
    t_end = time.perf_counter()
    # time the Hessian work took on its stream (with overlap: while quantization ran beside it), and the rest of the wall
    res.seconds["hessians_incl_gather_and_forward"] = ev0.elapsed_time(ev1) / 1e3
    res.seconds["quantize_and_pack"] = (t_end - t1) - res.seconds["hessians_incl_gather_and_forward"]
    res.overlapped = bool(overlap)
    issues = {"zero_samples": 0, "nan_hessian": 0, "non_invertible": 0}
    for name, h in done:
        raised = [k for k, v in (("zero_samples", h.issue_zero_samples), ("nan_hessian", h.issue_nan_hessian),
                                 ("non_invertible", h.issue_non_invertible)) if v]
        for k in raised:
            issues[k] += 1
        if raised:
            res.issues_by_linear[name] = raised
    res.factorizations = GPTQ.factor_calls - factor_calls_before
    res.seconds["total"] = time.perf_counter() - t0
    res.issues = issues
    return res
