#!/usr/bin/env python3
"""Benchmark of the GPTQ hot path on one MI355X.

One step = one pass of the whole path over config 1 (single expert gate_proj, 2048x7168 bf16 weights,
8192x7168 bf16 calibration tokens with 1% outlier channels, 4-bit symmetric, group 128, block 128):
Hessian accumulation -> damped factorisation -> GPTQ column loop -> packed int32 words + bf16 scales.
All inputs are resident in HBM before the timed region starts.  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

R_, C_, N_ = 2048, 7168, 8192
PEAK_FP32_MFMA = 157.3  # TFLOP/s, MI355X dense fp32 matrix
PEAK_BF16_MFMA = 2500.0  # TFLOP/s, MI355X dense bf16 matrix
PEAK_HBM = 8000.0  # GB/s


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=96)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--streams", type=int, default=3,
                    help="groups of independent linears are queued round-robin on this many HIP streams")
    ap.add_argument("--group", type=int, default=16,
                    help="independent linears per grouped library call (1 = one linear per call, as a lone GPTQ handle runs)")
    ap.add_argument("--moe-group", type=int, default=8, help="experts per grouped call in the MoE-layer workload")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--scale", type=float, default=1.0, help="shrink config 1 (debug only; 1.0 is the benchmark)")
    ap.add_argument("--workload", default="config1", choices=["config1", "config2", "config4", "config5", "moe_layer", "gemm", "syrk", "overlap"],
                    help="config1 (default, the benchmark line), config2 / config4 / config5 (the linears of those configurations, "
                         "one at a time as a block's non-expert linears run), moe_layer (config 3: whole MoE layer, one pass) or gemm "
                         "(micro-benchmark of the fp32 GEMM core shared by the factorisation and the loop) or syrk (the "
                         "Hessian kernel beside the vendor library's GEMM on the same operands) or overlap (how far grouped calls on "
                         "different HIP streams run beside each other)")
    ap.add_argument("--experts", type=int, default=256)
    ap.add_argument("--tokens", type=int, default=2_097_152)
    ap.add_argument("--check-experts", type=int, default=2, help="moe_layer: experts compared with the CPU oracle")
    ap.add_argument("--no-overlap", action="store_true",
                    help="moe_layer: the reference's order, every Hessian of the layer first, then quantization (kernel "
                         "durations in a profiler trace are then not stretched by kernels of the other streams)")
    ap.add_argument("--only", default=None, help="config4 / config5: run just the linear of this name (e.g. o_proj, down_g128)")
    ap.add_argument("--plain", action="store_true",
                    help="config2 / config4 / config5: whole steps only (one warm-up + --reps), no per-phase timing passes")
    ap.add_argument("--reps", type=int, default=0, help="config2 / config4 / config5: timed repetitions per linear (0 = default)")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="config1: skip the lone linears of configs 2, 4 and 5 reported next to the headline")
    ap.add_argument("--no-moe-layer", action="store_true",
                    help="config1: skip the one pass over the whole MoE layer (config 3) reported next to the headline")
    return ap.parse_args()


def kernel_sources_sha():
    """Short hash over the library's kernel sources: a profile table records it, so that a table made for other kernels
    than the ones running shows up in the line that quotes it."""
    import hashlib

    h = hashlib.sha1()
    d = os.path.join(ROOT, "moe_quant_amd", "csrc")
    for f in sorted(os.listdir(d)):
        if f.endswith((".hip", ".hpp")):
            h.update(f.encode())
            h.update(open(os.path.join(d, f), "rb").read())
    return h.hexdigest()[:12]


def profile_sources_sha(file="config1_bench_hbm_traffic"):
    """The kernel-source hash recorded in profiles/<file>.md (a line `kernel sources: <hash>`), or None."""
    path = os.path.join(ROOT, "profiles", file + ".md")
    if not os.path.exists(path):
        return None
    for line in open(path):
        if line.startswith("kernel sources:"):
            return line.split(":", 1)[1].strip()
    return None


def traffic_from_profiles(call, file="config1_bench_hbm_traffic", **keys):
    """HBM bytes per call of `call` for the configuration `keys`, from the table of measured traffic committed in
    profiles/<file>.md (lines of the form `| call | C=7168 G=8 panels=8 | 2.4e10 | ...`, made by rocprofv3 --pmc runs of
    this script); None if that table has no such line."""
    path = os.path.join(ROOT, "profiles", file + ".md")
    if not os.path.exists(path):
        return None
    want = " ".join(f"{k}={v}" for k, v in keys.items())
    for line in open(path):
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if len(cells) >= 3 and cells[0] == call and cells[1] == want:
            try:
                return float(cells[2])
            except ValueError:
                return None
    return None


def _timed(fn, reps=3, warm=1):
    """Mean device time of fn() in ms: HIP events on the stream the library launches on (torch's current stream)."""
    import torch

    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def device_inputs(dev, R, C, n, seed, x_kind="outlier"):
    """W (R,C) bf16 ~ N(0, 0.02^2) and X (n,C) bf16 drawn in HBM: N(0,1) tokens with 1% of the channels x20
    ("outlier"), or SiLU(a)*b with a, b ~ N(0,1) ("swiglu", the input of a down projection)."""
    import torch

    from moe_quant_amd import synth

    gen = torch.Generator(device=dev).manual_seed(seed)
    W = (torch.randn(R, C, generator=gen, device=dev) * 0.02).to(torch.bfloat16)
    X = torch.empty(n, C, dtype=torch.bfloat16, device=dev)
    outl = synth.outlier_channels(C, seed + 1).to(dev)
    for s0 in range(0, n, 16384):
        m = min(16384, n - s0)
        a = torch.randn(m, C, generator=gen, device=dev)
        if x_kind == "swiglu":
            a = torch.nn.functional.silu(a) * torch.randn(m, C, generator=gen, device=dev)
        else:
            a[:, outl] *= 20.0
        X[s0:s0 + m] = a.to(torch.bfloat16)
    return W, X


PLAIN = [False]  # --plain: the lone-linear workloads run whole steps only (one warm-up + reps), for profiler runs


def linear_leg(dev, name, R, C, n, g, act_order, x_kind="outlier", seed=0, reps=3, profile_key=None):
    """One linear quantized alone on the GPU -- the regime of a block's attention, dense-MLP and shared-expert linears,
    which the reference quantizes one by one (quant.py:291-330) and which have no sibling of the same shape to share
    grouped calls with.  Returns wall times of the whole step (Hessian -> packed words) and of H ready -> packed words,
    the device time of every phase (HIP events on the launch stream), the three big phases against their yardsticks
    and a `roofline` object for the phase that takes longest."""
    import torch

    from moe_quant_amd import ops
    from moe_quant_amd.gptq import GPTQ

    W, X = device_inputs(dev, R, C, n, seed, x_kind)
    layer = torch.nn.Linear(C, R, bias=False, dtype=torch.bfloat16, device=dev)
    layer.weight.data = W
    order = "activation" if act_order else "default"
    make = lambda: GPTQ(layer, group_size=g, sym=True, rel_damp=0.01, block_size=128, quantization_order=order)

    def whole():
        h = make()
        h.update(X)
        out = h.quantize(4)
        return h, out, h.packed_words()

    whole()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        last = whole()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / reps
    assert not last[0].has_hessian_issues()
    del last
    if PLAIN[0]:
        return {"linear": name, "R": R, "C": C, "tokens": n, "group_size": g, "act_order": bool(act_order),
                "ms_hessian_to_packed": round(ms_step, 3), "whole_steps_run": reps + 1, "roofline": None}
    hs = [make() for _ in range(reps)]
    for h in hs:
        h.update(X)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for h in hs:
        h.quantize(4)
        h.packed_words()
    torch.cuda.synchronize()
    ms_quant = (time.perf_counter() - t0) * 1e3 / reps
    del hs
    torch.cuda.empty_cache()

    # ---- phases, each call timed by itself
    H = torch.empty(C, C, device=dev)
    t_syrk = _timed(lambda: ops.hessian_syrk_(H, X, 0.0, 2.0 / n, mirror=False), reps)
    t_prestep = _timed(lambda: ops.hessian_prestep_(H, True), reps)
    t_perm, Hp, perm32, pinv32 = 0.0, H, None, None
    if act_order:
        def permute():
            perm = torch.argsort(H.diag(), descending=True)
            pinv = torch.argsort(perm)
            return ops.permute_symmetric(H, perm.to(torch.int32)), perm, pinv

        t_perm = _timed(permute, reps)
        Hp, perm, pinv = permute()
        perm32, pinv32 = perm.to(torch.int32), pinv.to(torch.int32)
    flags = torch.zeros(4, dtype=torch.int32, device=dev)
    Hs = Hp.clone()
    t_damp = _timed(lambda: ops.hessian_damp_(Hs, W, None, 0.01, flags), reps)  # (scratch copy: damped again every time)
    del Hs
    Hd = Hp.clone()
    ops.hessian_damp_(Hd, W, None, 0.01, flags)
    t_factor = _timed(lambda: ops.factor_chol(Hd), reps)
    F, info = ops.factor_chol(Hd)
    t_grid = _timed(lambda: ops.quant_grid_sym(W, g, 4, torch.bfloat16), reps)
    s_rg, s_gr = ops.quant_grid_sym(W, g, 4, torch.bfloat16)
    cols = perm if act_order else torch.arange(C, device=dev)
    scale_row = (cols // g).to(torch.int32)
    t_prep = _timed(lambda: ops.prepare_wt_pair(W, perm32), reps)
    Wt, W0t = ops.prepare_wt_pair(W, perm32)
    t_wcopy = _timed(lambda: Wt.copy_(W0t), reps)
    loop = lambda: ops.gptq_loop_chol_grouped_([Wt], [W0t], [F], [s_gr], [scale_row], 8.0, 15.0, torch.bfloat16, 128)[0]
    t_loop = _timed(lambda: (Wt.copy_(W0t), loop()), reps) - t_wcopy
    Qt = loop()
    t_untr = _timed(lambda: ops.untranspose_codes(Qt, pinv32), reps)
    t_pack = _timed(lambda: ops.pack_from_qt(Qt, pinv32), reps)
    assert int(info.item()) == 0
    flop = {"hessian_syrk": float(n) * C * (C + 1), "factor_chol": C**3 / 3.0, "gptq_loop": float(R) * C * (C - 1)}
    ms = {"hessian_syrk": t_syrk, "factor_chol": t_factor, "gptq_loop": t_loop}
    peak = {"hessian_syrk": PEAK_BF16_MFMA, "factor_chol": PEAK_FP32_MFMA, "gptq_loop": PEAK_FP32_MFMA}
    frac = {k: flop[k] / ms[k] / 1e9 / peak[k] for k in ms}
    dom = max(ms, key=ms.get)
    entry = {"hessian_syrk": "mq_hessian_syrk", "factor_chol": "mq_factor_chol", "gptq_loop": "mq_gptq_loop_chol"}[dom]
    unit_note = {
        "hessian_syrk": "algorithmic n*C*(C+1) flop (upper triangle) against the bf16 matrix peak",
        "factor_chol": "algorithmic C^3/3 flop (one Cholesky factorisation: the inverse-free loop needs no triangular "
                       "inverse, so this is half of the (2/3)C^3 a factor of the inverse costs) against the fp32 matrix "
                       "figure; the GEMM tiles run six bf16-piece products per fp32 product on the bf16 pipes",
        "gptq_loop": "algorithmic R*C*(C-1) flop against the fp32 matrix figure; trailing tiles run six bf16-piece "
                     "products per fp32 product on the bf16 pipes",
    }[dom]
    traffic = traffic_from_profiles(entry, file=profile_key, C=C, R=R, n=n) if profile_key else None
    out = {
        "linear": name, "R": R, "C": C, "tokens": n, "group_size": g, "act_order": bool(act_order),
        "ms_hessian_to_packed": round(ms_step, 3),
        "ms_h_ready_to_packed": round(ms_quant, 3),
        "phases_ms": {
            "hessian_syrk": round(t_syrk, 4), "prestep_mirror_scan": round(t_prestep, 4),
            "act_order_sort_and_gather": round(t_perm, 4), "damp": round(t_damp, 4), "factor_chol": round(t_factor, 4),
            "grid": round(t_grid, 4), "prepare_wt_pair": round(t_prep, 4), "gptq_loop": round(t_loop, 4),
            "untranspose_codes": round(t_untr, 4), "pack_from_loop_codes": round(t_pack, 4),
        },
        "hessian_syrk_tflops": round(flop["hessian_syrk"] / t_syrk / 1e9, 1),
        "hessian_syrk_frac_bf16_peak": round(frac["hessian_syrk"], 4),
        "factor_chol_tflops": round(flop["factor_chol"] / t_factor / 1e9, 2),
        "factor_chol_frac_fp32_mfma": round(frac["factor_chol"], 4),
        "gptq_loop_tflops": round(flop["gptq_loop"] / t_loop / 1e9, 2),
        "gptq_loop_frac_fp32_mfma": round(frac["gptq_loop"], 4),
        "pack_gbps": round(1.5 * R * C / t_pack / 1e6, 1),
        "roofline": {
            "kernel": f"{entry}, one linear per call ({name}: R={R} C={C} n={n}); {unit_note}",
            "bound": "mfma", "achieved": round(flop[dom] / ms[dom] / 1e9, 3), "peak": peak[dom], "unit": "TFLOP/s",
            "frac": round(frac[dom], 4), "traffic": traffic,
            "algorithmic_flop_per_launch": flop[dom], "ms_per_launch": round(ms[dom], 4),
        },
    }
    del H, Hp, Hd, F, Wt, W0t, Qt, X, W
    torch.cuda.empty_cache()
    return out


def cpu_linear_sample(R, C, n, g, act_order, x_kind, Rs, Cs, ns, seed=7):
    """The torch CPU oracle (the restated reference path) on a bounded sample of one linear: Rs rows, Cs input channels,
    ns tokens of the same distributions; Hessian product, the three-call Cholesky chain and the column loop are timed
    separately and each is scaled to the full linear by its flop count (n*C^2, C^3, R*C*(C-1))."""
    import torch

    from moe_quant_amd import synth
    from oracle import gptq_oracle as O

    torch.set_num_threads(min(16, os.cpu_count() or 1))
    Rs, Cs, ns = min(R, Rs), min(C, Cs), min(n, ns)
    W = synth.weight(Rs, Cs, seed)
    X = synth.activations_swiglu(ns, Cs, seed + 1) if x_kind == "swiglu" else synth.activations_outlier(ns, Cs, seed + 1)
    t0 = time.perf_counter()
    H, _ = O.hessian_update(None, 0, X)
    t_h = time.perf_counter() - t0
    H, W32, _, _ = O.quantization_pre_step(H, W)
    sc, zz, maxq = O.quantization_grid(W32, g, 4, torch.bfloat16)
    sr, zr = O.replicate_grid(sc, zz, g)
    perm, pinv = O.act_order_perm(H, act_order)
    H = H[perm][:, perm]
    t0 = time.perf_counter()
    U, ok = O.hessian_inverse(H, W32, 0.01)
    t_c = time.perf_counter() - t0
    Wt = W32.t()[perm].contiguous()
    st, zt = sr.t()[perm].contiguous(), zr.t()[perm].contiguous()
    t0 = time.perf_counter()
    q = O.gptq_loop(Wt, U, st, zt, maxq, torch.bfloat16, 128)
    O.pack_to_int32(q[pinv].t().contiguous().to(torch.int8) - 8, 4)
    t_l = time.perf_counter() - t0
    k_h = (float(n) * C * C) / (float(ns) * Cs * Cs)
    k_c = (C / Cs) ** 3
    k_l = (float(R) * C * (C - 1)) / (float(Rs) * Cs * (Cs - 1))
    full = t_h * k_h + t_c * k_c + t_l * k_l
    exact = (Rs, Cs, ns) == (R, C, n)
    return {
        "value": round(full, 3), "unit": "s per linear (Hessian + 3-call Cholesky chain + column loop + pack)",
        "cores": torch.get_num_threads(), "kind": "port",
        "sample": (f"the whole linear ({R}x{C}, {n} tokens)" if exact else
                   f"a {Rs}x{Cs} linear with {ns} tokens of the same distributions, measured {t_h + t_c + t_l:.1f} s "
                   f"(Hessian {t_h:.2f}, chain {t_c:.2f}, loop+pack {t_l:.2f}); EXTRAPOLATED to {R}x{C}, {n} tokens by flop "
                   f"count (factors {k_h:.1f}, {k_c:.1f}, {k_l:.1f})"),
        "measured_s": {"hessian": round(t_h, 3), "cholesky_chain": round(t_c, 3), "loop_and_pack": round(t_l, 3)},
        "extrapolated": not exact, "host_cpu_count": os.cpu_count(),
    }


def moe_layer_run(args, with_cpu_oracle=True):
    """Config 3: every Hessian of a DeepSeek-V3-shaped MoE layer accumulated, 3 linears per expert quantized
    and packed, on one GPU, one pass.  Returns a dict of wall seconds, sizes and (optionally) the parity of the
    busiest experts' linears against the CPU oracle."""
    import torch

    from moe_quant_amd import _lib, synth
    from moe_quant_amd.moe_layer import ExpertWeights, quantize_moe_layer

    _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    t0 = time.perf_counter()
    x, ids, ex = synth.moe_layer_on_device(dev, args.experts, args.tokens)
    torch.cuda.synchronize()
    t_gen = time.perf_counter() - t0
    experts = [ExpertWeights(*w) for w in ex]
    # warm-up on a tiny problem so that one-time costs (module load, allocator growth) stay out of the clock
    quantize_moe_layer(x[:4096], ids[:4096] % 2, experts[:2])
    counts = torch.bincount(ids.flatten(), minlength=args.experts)
    check = torch.argsort(counts, descending=True)[: args.check_experts].tolist() if args.check_experts else []
    res = quantize_moe_layer(x, ids, experts, keep_codes=check, overlap=not getattr(args, "no_overlap", False),
                             group=getattr(args, "moe_group", 8))
    C, I = x.shape[1], experts[0].gate.shape[0]
    n_e = torch.tensor(res.tokens_per_expert, dtype=torch.float64)
    flop_syrk = float((n_e * (C * (C + 1) + I * (I + 1))).sum())
    out = {
        "wall_s": round(res.seconds["total"], 3),
        "seconds": {k: round(v, 3) for k, v in res.seconds.items()},
        "quantization_overlaps_hessian_collection": res.overlapped,
        "experts": args.experts, "tokens": args.tokens, "top_k": int(ids.shape[1]), "hidden": C, "inter": I,
        "linears": 3 * args.experts,
        "generate_inputs_s": round(t_gen, 2),
        "tokens_per_expert": {"min": int(n_e.min()), "max": int(n_e.max()), "mean": float(n_e.mean())},
        "hessian_algorithmic_tflop": round(flop_syrk / 1e12, 1),
        "issues": res.issues,
        "note": "seconds.hessians_... is the time of the Hessian stream (token gather, expert forward, SYRK) with the "
                "quantization of earlier experts running beside it, seconds.quantize_and_pack the rest of the wall; "
                "seconds.hessians counts the expert forward (gate/up products + SiLU product) that produces the "
                "down-projection inputs; the model forward is not part of the GPTQ kernels' rooflines",
    }
    if check and with_cpu_oracle:
        from oracle import gptq_oracle as O

        torch.set_num_threads(min(16, os.cpu_count() or 1))
        par = {}
        t_cpu = 0.0
        for e in check:
            for proj, w in (("gate_proj", experts[e].gate), ("down_proj", experts[e].down)):
                Hc = res.hessians[f"{e}.{proj}"].cpu()
                tc = time.perf_counter()
                ref = O.quantize_linear(w.cpu(), Hc)
                t_cpu += time.perf_counter() - tc
                q = res.qweight[f"{e}.{proj}"].cpu()
                n_tok = res.tokens_per_expert[e]
                par[f"{e}.{proj}"] = {
                    "code_match": round((q == ref["qweight"]).float().mean().item(), 6),
                    # the oracle runs on the very Hessian the GPU accumulated: what is compared is factorisation + loop
                    "hessian": "the GPU's (same matrix on both sides)",
                    "tokens": n_tok,
                    # experts with fewer tokens than input channels have a singular Hessian held up by damping alone;
                    # the test suite gates those at the oracle's own measured floor minus 0.2% instead of 99.9%
                    "gate": 0.999 if n_tok >= w.shape[1] else "relaxed: oracle-against-itself floor - 0.002 (tests/test_gpu_moe_layer.py)",
                    "scales_equal": bool(torch.equal(res.scales[f"{e}.{proj}"].cpu(), ref["scale"])),
                }
        out["parity_vs_cpu_oracle"] = par
        out["cpu_baseline"] = {
            "value": round(t_cpu / (2 * len(check)), 3), "unit": "s per linear (quantize only, Hessian given)",
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{2 * len(check)} linears of the layer (gate and down of the {len(check)} busiest experts), "
                      f"extrapolated layer quantize time = {t_cpu / (2 * len(check)) * 3 * args.experts:.0f} s",
        }
    del x, ids, ex, experts, res
    torch.cuda.empty_cache()
    return out


def moe_layer_main(args):
    """`--workload moe_layer`: prints one JSON line whose metric is the MoE-layer wall time."""
    r = moe_layer_run(args, with_cpu_oracle=not args.no_cpu_baseline)
    out = {
        "metric": "MoE-layer wall seconds (256 experts x 3 linears, 2M routed calibration tokens)",
        "value": r["wall_s"],
        "unit": "s",
        "n_gpus": 1,
        "steps": 1,
        "warmup": 0,
        "ms_per_step": round(r["wall_s"] * 1e3, 1),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "config 3: DeepSeek-V3-shaped MoE layer, all Hessians resident, GPTQ 4-bit g128 on all linears",
                   "experts": r["experts"], "tokens": r["tokens"], "top_k": r["top_k"], "hidden": r["hidden"],
                   "inter": r["inter"], "linears": r["linears"]},
    }
    out.update({k: v for k, v in r.items() if k not in ("experts", "tokens", "top_k", "hidden", "inter", "linears", "wall_s")})
    print(json.dumps(out))


def gemm_main(args):
    """Micro-benchmark of mq_gemm_f32 (fp32 in and out; interior tiles form each product from six bf16-piece products
    on the bf16 matrix cores): the shapes the factorisation and the loop issue.  One JSON line, TFLOP/s per shape."""
    import torch

    from moe_quant_amd import _lib, ops

    _lib.load()
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(0)
    shapes = [(4096, 4096, 4096, 0.0), (8192, 8192, 128, 1.0), (8192, 8192, 256, 1.0), (8192, 8192, 512, 1.0),
              (8192, 8192, 1024, 1.0), (7040, 2048, 128, 1.0), (6656, 2048, 512, 1.0)]
    out = {}
    for M, N, K, beta in shapes:
        A = torch.randn(M, K, generator=g, device=dev)
        Bm = torch.randn(N, K, generator=g, device=dev)  # B(k,n) = Bm[n,k]: both operands K-contiguous
        Cm = torch.zeros(M, N, device=dev)
        run = lambda: ops.gemm_f32_(A, K, 1, Bm, 1, K, Cm, M, N, K, alpha=1.0, beta=beta)
        for _ in range(3):
            run()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        reps = 20
        e0.record()
        for _ in range(reps):
            run()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        out[f"{M}x{N}x{K} beta={beta:g}"] = {"ms": round(ms, 4), "tflops": round(2.0 * M * N * K / ms / 1e9, 1)}
    print(json.dumps({"metric": "fp32 GEMM core TFLOP/s (fp32 in/out, six bf16-piece products per fp32 product)",
                      "unit": "TFLOP/s", "n_gpus": 1, "dtype": "f32", "data": "synthetic", "peak_fp32_mfma": PEAK_FP32_MFMA,
                      "shapes": out}))


def syrk_main(args):
    """The Hessian kernel (upper triangle only, tokens read as the hooks deliver them: token-major) beside the vendor
    GEMM torch dispatches for X^T X on the same tensor (full product), and beside the same GEMM on a pre-transposed
    copy (both operands contiguous along the tokens, the layout matrix cores like best).  One JSON line."""
    import torch

    from moe_quant_amd import _lib, ops

    _lib.load()
    dev = torch.device("cuda:0")

    def timed(fn, reps=8):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    out = {}
    for n, C in ((8192, 7168), (32768, 7168), (131072, 7168), (65536, 2048)):
        X = torch.randn(n, C, device=dev).to(torch.bfloat16)
        H = torch.zeros(C, C, device=dev)
        alg = n * C * (C + 1)
        t_own = timed(lambda: ops.hessian_syrk_(H, X, 0.0, 2.0 / n, mirror=False))
        Xp = ops.pack_tokens(X)
        t_pack = timed(lambda: ops.pack_tokens(X))
        Hp = torch.zeros(C, C, device=dev)
        t_packed = timed(lambda: ops.hessian_syrk_packed_(Hp, Xp, 0.0, 2.0 / n, mirror=False))
        same = bool(torch.equal(torch.triu(Hp), torch.triu(H)))
        rel = ((torch.triu(Hp) - torch.triu(H)).norm() / torch.triu(H).norm()).item()
        del Xp, Hp
        t_lib = timed(lambda: X.t() @ X)
        Xt = X.t().contiguous()
        t_lib_t = timed(lambda: Xt @ Xt.t())
        out[f"n={n} C={C}"] = {
            "mq_hessian_syrk_ms": round(t_own, 4), "algorithmic_tflops": round(alg / t_own / 1e9, 1),
            "frac_bf16_peak": round(alg / t_own / 1e9 / PEAK_BF16_MFMA, 4),
            "mq_hessian_syrk_packed_ms": round(t_packed, 4), "packed_algorithmic_tflops": round(alg / t_packed / 1e9, 1),
            "mq_pack_tokens_ms": round(t_pack, 4), "pack_gbps": round(4.0 * n * C / t_pack / 1e6, 1),
            "packed_equals_token_major_bits": same, "packed_vs_token_major_rel_diff": rel,
            "vendor_gemm_same_layout_ms": round(t_lib, 4),
            "vendor_gemm_same_layout_executed_tflops": round(2.0 * n * C * C / t_lib / 1e9, 1),
            "vendor_gemm_pretransposed_ms": round(t_lib_t, 4),
            "vendor_gemm_pretransposed_executed_tflops": round(2.0 * n * C * C / t_lib_t / 1e9, 1),
        }
        del X, Xt, H
    print(json.dumps({"metric": "Hessian SYRK TFLOP/s (algorithmic n*C*(C+1)) beside the vendor GEMM on the same operands",
                      "unit": "TFLOP/s", "n_gpus": 1, "dtype": "bf16", "data": "synthetic", "peak_bf16_mfma": PEAK_BF16_MFMA,
                      "shapes": out}))


def overlap_main(args):
    """How far library calls queued on different HIP streams run beside each other on the chip: every phase of
    config 1 as grouped calls of eight, six calls dealt round-robin to 1..4 streams; then a call that is one chain of
    short launches (a lone factorisation, a lone column loop) beside calls that fill the chip (grouped SYRK, grouped
    factorisation), alone and together.  One JSON line."""
    import time

    import torch

    from moe_quant_amd import _lib, ops

    _lib.load()
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    C, R, n, G, NB = 7168, 2048, 8192, 8, 6
    X = [torch.randn(n, C, device=dev).to(torch.bfloat16) for _ in range(G)]

    def hessians():
        Hs = [torch.zeros(C, C, device=dev) for _ in range(G)]
        ops.hessian_syrk_grouped_(Hs, X, [0.0] * G, [2.0 / n] * G)
        for H in Hs:
            H.diagonal().add_(0.01 * H.diagonal().mean())
        return Hs

    Hb = [hessians() for _ in range(NB)]
    H1 = [Hb[0][0].clone() for _ in range(8)]
    W = [(torch.randn(R, C, device=dev) * 0.02).to(torch.bfloat16) for _ in range(G)]
    Fs, _ = ops.factor_chol_grouped([h.clone() for h in Hb[0]])
    scales = [ops.quant_grid_sym(w, 128, 4, torch.bfloat16)[1] for w in W]
    srow = [torch.arange(C, device=dev, dtype=torch.int32) // 128 for _ in range(G)]
    pairs = [[ops.prepare_wt_pair(w) for w in W] for _ in range(NB)]
    lone = [ops.prepare_wt_pair(W[0]) for _ in range(10)]

    def syrk(b):
        ops.hessian_syrk_grouped_(Hb[b % NB], X, [0.0] * G, [2.0 / n] * G)

    def chol(b):
        ops.factor_chol_grouped(Hb[b % NB])

    def loop(b):
        ops.gptq_loop_chol_grouped_([p[0] for p in pairs[b % NB]], [p[1] for p in pairs[b % NB]], Fs, scales, srow, 8.0, 15.0,
                                    torch.bfloat16, 128)

    def chol1(i):
        ops.factor_chol(H1[i % 8])

    def loop1(i):
        ops.gptq_loop_chol_grouped_([lone[i % 10][0]], [lone[i % 10][1]], [Fs[0]], [scales[0]], [srow[0]], 8.0, 15.0,
                                    torch.bfloat16, 128)

    streams = [torch.cuda.Stream(device=dev) for _ in range(4)]

    def wall(plan):  # plan: (function, argument, stream index); best of three after one untimed pass
        best = None
        for it in range(4):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for fn, a, si in plan:
                with torch.cuda.stream(streams[si]):
                    fn(a)
            torch.cuda.synchronize()
            t = (time.perf_counter() - t0) * 1e3
            if it and (best is None or t < best):
                best = t
        return round(best, 2)

    out = {"ms_per_linear_by_streams": {}, "chain_beside_full_chip_ms": {}}
    kinds = {"syrk": [syrk], "factor": [chol], "loop": [loop], "factor+loop": [chol, loop], "syrk+factor+loop": [syrk, chol, loop]}
    for name, fns in kinds.items():
        calls = [(f, b) for b in range(NB) for f in fns]
        out["ms_per_linear_by_streams"][name] = {
            str(S): round(wall([(f, b, i % S) for i, (f, b) in enumerate(calls)]) / (NB * G), 3) for S in (1, 2, 3, 4)}
    for (na, fa, ca), (nb_, fb, cb) in ((("syrk x8", syrk, 6), ("lone factor", chol1, 7)),
                                        (("syrk x8", syrk, 6), ("lone loop", loop1, 10)),
                                        (("factor x8", chol, 3), ("lone factor", chol1, 7)),
                                        (("factor x8", chol, 3), ("lone loop", loop1, 10))):
        a = wall([(fa, i, 0) for i in range(ca)])
        b = wall([(fb, i, 1) for i in range(cb)])
        ab = wall([(fa, i, 0) for i in range(ca)] + [(fb, i, 1) for i in range(cb)])
        out["chain_beside_full_chip_ms"][f"{ca} calls of {na} | {cb} calls of {nb_}"] = {"first_alone": a, "second_alone": b, "together": ab}
    print(json.dumps({"metric": "wall time of config-1 library calls queued on several HIP streams", "unit": "ms", "n_gpus": 1,
                      "data": "synthetic", "linears_per_grouped_call": G, **out}))


CONFIG4_SHAPES = {"q_a_proj": (1536, 7168), "q_b_proj": (24576, 1536), "kv_a_proj_with_mqa": (576, 7168),
                  "kv_b_proj": (32768, 512), "o_proj": (7168, 16384)}


def config2_run(dev, cpu, reps=5):
    """Config 2: expert down_proj 7168x2048, 65536 SwiGLU tokens, 4-bit g128, packed words + bf16 scales."""
    leg = linear_leg(dev, "down_proj", 7168, 2048, 65536, 128, False, "swiglu", seed=2, reps=reps, profile_key="config2_hbm_traffic")
    if cpu:
        leg["cpu_baseline"] = cpu_linear_sample(7168, 2048, 65536, 128, False, "swiglu", 7168, 2048, 65536)
    return leg


def config4_run(dev, cpu, reps=3, cpu_full=False, only=None):
    """Config 4: the five MLA attention linears, 16384 tokens per input width, one at a time."""
    legs = {}
    for i, (name, (R, C)) in enumerate(CONFIG4_SHAPES.items()):
        if only and name != only:
            continue
        legs[name] = linear_leg(dev, name, R, C, 16384, 128, False, "outlier", seed=40 + i, reps=reps,
                                profile_key="config4_hbm_traffic")
    if cpu and "o_proj" in legs:
        # one bounded sample: o_proj, the linear that decides the block's attention part (16384^2 Hessian)
        Cs = 16384 if cpu_full else 4096
        legs["o_proj"]["cpu_baseline"] = cpu_linear_sample(7168, 16384, 16384, 128, False, "outlier", 512 if cpu_full else 2048,
                                                           Cs, 2048 if cpu_full else 4096)
    return legs


def config5_run(dev, cpu, reps=2, groups=(128, 64, 32), cpu_full=False, only=None):
    """Config 5: dense MLP with act-order, gate/up 18432x7168 and down 7168x18432, 65536 tokens, g in {128, 64, 32}."""
    legs = {}
    for g in groups:
        if not only or only == f"gate_up_g{g}":
            legs[f"gate_up_g{g}"] = linear_leg(dev, f"gate_up g{g}", 18432, 7168, 65536, g, True, "outlier", seed=50,
                                               reps=reps, profile_key="config5_hbm_traffic")
        if not only or only == f"down_g{g}":
            legs[f"down_g{g}"] = linear_leg(dev, f"down g{g}", 7168, 18432, 65536, g, True, "outlier", seed=51, reps=reps,
                                            profile_key="config5_hbm_traffic")
    if cpu and f"down_g{groups[0]}" in legs:
        Cs = 18432 if cpu_full else 4096
        legs[f"down_g{groups[0]}"]["cpu_baseline"] = cpu_linear_sample(7168, 18432, 65536, groups[0], True, "outlier",
                                                                       256 if cpu_full else 2048, Cs, 1024 if cpu_full else 4096)
    return legs


def _leg_line(metric, workload, legs, head=None):
    """One JSON line for a workload made of lone linears: value = linears/s over all of them, roofline and cpu_baseline
    of the linear `head` (the one the configuration is there to stress)."""
    if head is None:
        legs, head = legs
    total_ms = sum(l["ms_hessian_to_packed"] for l in legs.values())
    line = {
        "metric": metric, "value": round(len(legs) * 1000.0 / total_ms, 3), "unit": "linears/s", "n_gpus": 1,
        "steps": len(legs), "warmup": 1, "ms_per_step": round(total_ms / len(legs), 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": workload, "linears": list(legs), "one_linear_per_call": True},
        "roofline": legs[head]["roofline"], "cpu_baseline": legs[head].get("cpu_baseline"),
        "linears": legs,
    }
    print(json.dumps(line))


def other_config_main(args):
    import torch

    from moe_quant_amd import _lib

    _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    cpu = not args.no_cpu_baseline and not args.plain
    PLAIN[0] = bool(args.plain)
    rp = lambda d: args.reps if args.reps > 0 else d
    if args.workload == "config2":
        leg = config2_run(dev, cpu, reps=rp(5))
        _leg_line("GPTQ linears/sec (7168x2048 expert down_proj, g128, packed)",
                  "config 2: expert down_proj 7168x2048 bf16, 65536 SwiGLU calibration tokens, 4-bit sym g128, packed int32 "
                  "words + bf16 scales; one linear per call", {"down_proj": leg}, "down_proj")
    elif args.workload == "config4":
        _leg_line("GPTQ linears/sec (MLA attention linears, g128)",
                  "config 4: q_a 1536x7168, q_b 24576x1536, kv_a 576x7168, kv_b 32768x512, o_proj 7168x16384, 16384 tokens per "
                  "input width, 4-bit sym g128; one linear per call",
                  (lambda legs: (legs, "o_proj" if "o_proj" in legs else next(iter(legs))))(
                      config4_run(dev, cpu, reps=rp(3), cpu_full=True, only=args.only)))
    else:
        legs = config5_run(dev, cpu, reps=rp(2), cpu_full=True, only=args.only)
        _leg_line("GPTQ linears/sec (dense MLP with act-order, g128/64/32)",
                  "config 5: gate/up 18432x7168 and down 7168x18432, 65536 tokens, act-order, 4-bit sym, group 128, 64 and 32; "
                  "one linear per call", (legs, "down_g128" if "down_g128" in legs else next(iter(legs))))


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this engine runs on one GPU (no sharding, no collectives); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    if args.workload == "moe_layer":
        return moe_layer_main(args)
    if args.workload == "gemm":
        return gemm_main(args)
    if args.workload == "syrk":
        return syrk_main(args)
    if args.workload == "overlap":
        return overlap_main(args)
    if args.workload in ("config2", "config4", "config5"):
        return other_config_main(args)
    import torch

    from moe_quant_amd import _lib, ops, synth
    from moe_quant_amd.gptq import GPTQ

    _lib.load()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    case = synth.config1(args.scale)
    R, C = case.W.shape
    n = case.X.shape[0]

    def layer_of(W):
        m = torch.nn.Linear(C, R, bias=False, dtype=torch.bfloat16, device=dev)
        m.weight.data.copy_(W)
        return m

    # Steps are independent linears.  One linear is a long chain of dependent launches that cannot fill the GPU by
    # itself, so `group` consecutive steps share grouped library calls (every launch carries the work of all of
    # them) and the groups go round-robin onto `streams` HIP streams; nothing in a step reads a value back, the
    # host just queues.
    main_stream = torch.cuda.current_stream(dev)
    n_lanes = max(1, args.streams)
    group = max(1, args.group)
    lanes = [main_stream] + [torch.cuda.Stream(device=dev) for _ in range(n_lanes - 1)]  # the current stream is lane 0
    # Every linear of a grouped call has its own calibration tokens and its own weights, and every stream its own set
    # of them (as the experts of a block have): nothing the timed steps read is shared between linears in flight.
    # Linear 0 of stream 0 is the seeded config-1 case the CPU oracle is run on; the others are drawn in HBM from the
    # same distributions (same outlier channels).
    gen = torch.Generator(device=dev).manual_seed(1234)
    outl = synth.outlier_channels(C, 103).to(dev)

    def more_tokens():
        x = torch.randn(n, C, generator=gen, device=dev)
        x[:, outl] *= 20.0
        return x.to(torch.bfloat16)

    Xsets = [[more_tokens() for _ in range(group)] for _ in range(n_lanes)]
    layers = [[layer_of((torch.randn(R, C, generator=gen, device=dev) * 0.02).to(torch.bfloat16)) for _ in range(group)]
              for _ in range(n_lanes)]
    Xsets[0][0] = case.X.to(dev)
    layers[0][0] = layer_of(case.W)
    X = Xsets[0][0]
    layer = layers[0][0]

    def handles(g, lane):
        return [GPTQ(layers[lane][i], group_size=128, sym=True, rel_damp=0.01, block_size=128) for i in range(g)]

    def accumulate(hs, lane):
        if len(hs) == 1:
            hs[0].update(Xsets[lane][0])
        else:
            GPTQ.update_many(hs, Xsets[lane][: len(hs)])

    def quantize_and_pack(hs):
        outs = [hs[0].quantize(4)] if len(hs) == 1 else GPTQ.quantize_many(hs, 4)
        return outs, [h.packed_words() for h in hs]

    def steps(g, lane):
        """g steps: g independent linears, each with its own tokens, weights, Hessian, factor, codes and words."""
        hs = handles(g, lane)
        accumulate(hs, lane)
        return quantize_and_pack(hs)

    def batches(k, n_lanes, group):
        """k steps as grouped batches of at most `group`, the same number of batches on every lane and sizes as equal
        as possible (a short run must not end with one lane working through a last batch alone)."""
        if k <= 0:
            return []
        rounds = -(-k // (n_lanes * group))
        nb = min(k, rounds * n_lanes)
        return [k // nb + (1 if i < k % nb else 0) for i in range(nb)]

    def run(k, lanes, group=group, ready=None):
        """k steps dealt to the lanes; ready: handles whose Hessians are already accumulated (then a step is only
        H ready -> packed words), one list per batch."""
        for ln in lanes:
            if ln is not main_stream:
                ln.wait_stream(main_stream)
        last = None
        t_begin = time.perf_counter()
        for bi, size in enumerate(batches(k, len(lanes), group)):
            with torch.cuda.stream(lanes[bi % len(lanes)]):
                last = quantize_and_pack(ready[bi]) if ready is not None else steps(size, bi % len(lanes))
        host_ms[0] = (time.perf_counter() - t_begin) * 1e3 / max(k, 1)
        torch.cuda.synchronize()
        return last

    host_ms = [0.0]
    # set-up, before the warm-up steps: one batch of the timed region's size on every lane, so that each lane's scratch
    # buffers and the allocator's pools exist (a first allocation synchronises the device) -- not counted as steps
    prime = batches(args.steps, len(lanes), group)
    run(len(lanes) * max(prime), lanes, max(prime)) if prime else None
    run(args.warmup, lanes)
    t0 = time.perf_counter()
    run(args.steps, lanes)
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    host_issue_ms = host_ms[0]
    # The same steps from "H ready" to "packed words and scales ready" (pre-step, grid, factorisation, loop, packing):
    # the Hessians of all those linears are accumulated beforehand (205 MB each, so at most 96 steps are timed this way).
    k_ready = min(args.steps, 96)
    # Run twice and time the second pass: with every Hessian of the region alive, the buffers the quantization allocates
    # (factor, transposed weights, codes) do not come out of blocks the earlier steps freed, and the first pass would
    # time the allocator taking that memory from the device.
    for timed_pass in (False, True):
        ready = []
        for bi, size in enumerate(batches(k_ready, len(lanes), group)):
            with torch.cuda.stream(lanes[bi % len(lanes)]):
                hs = handles(size, bi % len(lanes))
                accumulate(hs, bi % len(lanes))
                ready.append(hs)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run(k_ready, lanes, ready=ready)
        ms_h_ready = (time.perf_counter() - t0) * 1e3 / k_ready
        if not timed_pass:
            del ready
    del ready
    torch.cuda.empty_cache()
    # one step through the same grouped calls whose first linear is the seeded case: what the CPU oracle is compared with
    (outs, packed) = steps(min(group, 2), 0)
    out_q, out_s = outs[0][0], outs[0][1]
    torch.cuda.synchronize()
    # the same step, one at a time on one stream: the latency of a single linear
    run(1, [main_stream], 1)
    t0 = time.perf_counter()
    run(3, [main_stream], 1)
    ms_single = (time.perf_counter() - t0) * 1e3 / 3

    # ---- per-phase device times (HIP events on the stream the kernels run on), outside the timed region
    timed = lambda fn, reps=3: _timed(fn, reps)
    H = torch.zeros(C, C, device=dev)
    t_syrk = timed(lambda: ops.hessian_syrk_(H, X, 0.0, 2.0 / n))
    Hd = H.clone()
    Hd.diagonal().add_(0.01 * Hd.diag().mean())
    A = torch.empty_like(Hd)
    info = torch.zeros(1, dtype=torch.int32, device=dev)

    def factor():
        A.copy_(Hd)
        ops.factor_upper_inverse_(A, info)

    t_copy = timed(lambda: A.copy_(Hd), reps=8)
    t_factor_inv = timed(factor, reps=8) - t_copy  # the reference's factor U (public _get_hessian_inverse path)
    # what the quantize path runs: the Cholesky factor alone, as the multipliers of the inverse-free loop
    t_factor = timed(lambda: ops.factor_chol(Hd), reps=8)
    F, _ = ops.factor_chol(Hd)
    Wd = layer.weight.data
    s_rg, s_gr = ops.quant_grid_sym(Wd, 128, 4, torch.bfloat16)
    scale_row = torch.arange(C, device=dev, dtype=torch.int32) // 128
    Wt0 = ops.prepare_wt(Wd)
    Wt = torch.empty_like(Wt0)
    t_wcopy = timed(lambda: Wt.copy_(Wt0))
    loop1 = lambda: ops.gptq_loop_chol_grouped_([Wt], [Wt0], [F], [s_gr], [scale_row], 8.0, 15.0, torch.bfloat16, 128)[0]
    t_loop = timed(lambda: (Wt.copy_(Wt0), loop1())) - t_wcopy
    Wt.copy_(Wt0)
    Qt = loop1()
    t_pack = timed(lambda: ops.pack_from_qt(Qt), reps=10)
    codes = ops.untranspose_codes(Qt)
    t_pack_rc = timed(lambda: ops.pack_int4(codes), reps=10)
    # one launch of 22 MB is launch latency; the kernel's own rate shows on sixteen linears' codes stacked into one launch
    codes16 = codes.repeat(16, 1)
    t_pack16 = timed(lambda: ops.pack_int4(codes16), reps=10)
    del codes16

    # the three big phases once more as the step runs them: one grouped library call over `group` linears on one
    # stream, every linear with its own tokens, Hessian, factor and weights; device time of the call / group
    Gq = max(group, 1)
    Hs = [torch.zeros(C, C, device=dev) for _ in range(Gq)]
    t_syrk_g = timed(lambda: ops.hessian_syrk_grouped_(Hs, Xsets[0][:Gq], [0.0] * Gq, [2.0 / n] * Gq, mirror=False)) / Gq
    for Hi in Hs:
        Hi.diagonal().add_(0.01 * Hi.diag().mean())
    t_factor_g = timed(lambda: ops.factor_chol_grouped(Hs), reps=4) / Gq
    Fs, _ = ops.factor_chol_grouped(Hs)
    del Hs
    W0ts = [ops.prepare_wt(layers[0][i].weight.data) for i in range(Gq)]
    Wts = [torch.empty_like(Wt0) for _ in range(Gq)]
    sgrs = [ops.quant_grid_sym(layers[0][i].weight.data, 128, 4, torch.bfloat16)[1] for i in range(Gq)]

    def loop_grouped():
        for w, w0 in zip(Wts, W0ts):
            w.copy_(w0)
        ops.gptq_loop_chol_grouped_(Wts, W0ts, Fs, sgrs, [scale_row] * Gq, 8.0, 15.0, torch.bfloat16, 128)

    t_loop_g = timed(loop_grouped) / Gq - t_wcopy
    del Wts, W0ts, Fs, sgrs
    torch.cuda.empty_cache()

    pts = torch.linspace(1, 0.2, 100, dtype=torch.float32, device=dev)
    s_try = s_rg.clone()
    t_mse = timed(lambda: ops.mse_scale_sym_(Wd, 128, pts, s_try, None, 8.0, 15.0, 2.4, torch.bfloat16))

    flop_syrk = n * C * (C + 1)
    flop_factor = (1.0 / 3.0) * C**3  # one Cholesky factorisation: all the quantize path needs (no inverse)
    flop_loop = R * C * (C - 1)
    bytes_pack = 1.5 * R * C
    phases = {
        "hessian_syrk_ms": round(t_syrk, 4),
        "factor_ms": round(t_factor, 4),
        "factor_with_inverse_ms_not_in_step": round(t_factor_inv, 4),
        "gptq_loop_ms": round(t_loop, 4),
        "pack_from_loop_codes_ms": round(t_pack, 4),
        "pack_int4_ms": round(t_pack_rc, 4),
        "mse_scale_search_ms_not_in_step": round(t_mse, 4),
        "linears_per_grouped_call": Gq,
        "hessian_syrk_ms_per_linear_grouped": round(t_syrk_g, 4),
        "factor_ms_per_linear_grouped": round(t_factor_g, 4),
        "gptq_loop_ms_per_linear_grouped": round(t_loop_g, 4),
        "hessian_syrk_frac_bf16_peak_grouped": round(flop_syrk / t_syrk_g / 1e9 / PEAK_BF16_MFMA, 4),
        "factor_tflops_grouped": round(flop_factor / t_factor_g / 1e9, 2),
        "gptq_loop_tflops_grouped": round(flop_loop / t_loop_g / 1e9, 2),
        "hessian_syrk_tflops": round(flop_syrk / t_syrk / 1e9, 2),
        "hessian_syrk_frac_bf16_peak": round(flop_syrk / t_syrk / 1e9 / PEAK_BF16_MFMA, 4),
        "factor_tflops": round(flop_factor / t_factor / 1e9, 2),
        "gptq_loop_tflops": round(flop_loop / t_loop / 1e9, 2),
        "pack_int4_gbps": round(bytes_pack / t_pack_rc / 1e6, 1),
        "pack_int4_frac_hbm_peak": round(bytes_pack / t_pack_rc / 1e6 / PEAK_HBM, 4),
        "pack_int4_gbps_16_linears_one_launch": round(16 * bytes_pack / t_pack16 / 1e6, 1),
        "pack_int4_frac_hbm_peak_16_linears_one_launch": round(16 * bytes_pack / t_pack16 / 1e6 / PEAK_HBM, 4),
    }
    # Dominant call of the step: the factorisation, as the step runs it -- one grouped call over `group` matrices
    # (one "launch" = one call = a fixed sequence of kernels, each carrying the work of all matrices).
    # achieved = algorithmic flop (one Cholesky factorisation per matrix, C^3/3) / device time of the call, measured
    # above with HIP events on the launch stream.  traffic = HBM bytes per call from the rocprofv3 --pmc runs
    # summarised in profiles/ (looked up by matrix size, group size and panel batch; null when that table has no
    # line for this configuration).
    panels = int(os.environ.get("MQ_PANELS", "8") or 8)
    traffic = traffic_from_profiles("mq_factor_chol_grouped", C=C, G=Gq, panels=panels)
    tf_factor_g = flop_factor / t_factor_g / 1e9
    roofline = {
        "kernel": f"mq_factor_chol_grouped over {Gq} matrices = trail_diag_kernel + panel_inv_kernel + revchol_diag_kernel + "
                  "chol_finalize_kernel (one launch sequence per call; largest share of the step). fp32 in, fp32 out. "
                  "Algorithmic unit: C^3/3 flop per matrix, ONE Cholesky factorisation -- half of the (2/3)C^3 (Cholesky + "
                  "triangular inverse) a factor of the inverse costs, because the column loop runs on the Cholesky factor "
                  "itself and the inverse is never formed.  The interior GEMM tiles form each fp32 product from six "
                  "bf16-piece products on the bf16 matrix cores, so the fp32 MFMA figure is the yardstick for the "
                  "algorithmic flop, not a ceiling of the kernel; frac_of_bf16_pipe prices the executed piece products "
                  "(6 x algorithmic) against the bf16 matrix peak",
        "bound": "mfma",
        "achieved": round(tf_factor_g, 3),
        "peak": PEAK_FP32_MFMA,
        "unit": "TFLOP/s",
        "frac": round(tf_factor_g / PEAK_FP32_MFMA, 4),
        "frac_of_bf16_pipe": round(6.0 * tf_factor_g / PEAK_BF16_MFMA, 4),
        "traffic": traffic,
        "traffic_source": "profiles/config1_bench_hbm_traffic.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this "
                          "command, looked up by C, group and panel batch; not re-measured by this run)",
        "traffic_table_made_for_these_kernel_sources": profile_sources_sha() == kernel_sources_sha(),
        "algorithmic_flop_per_launch": flop_factor * Gq,
        "ms_per_launch": round(t_factor_g * Gq, 4),
    }
    # the same two calls for one linear at a time (no sibling to share launches with): what ms_per_step_one_stream is made of
    roofline_lone = {
        "mq_factor_chol": {"achieved": round(flop_factor / t_factor / 1e9, 2), "peak": PEAK_FP32_MFMA, "unit": "TFLOP/s",
                           "frac": round(flop_factor / t_factor / 1e9 / PEAK_FP32_MFMA, 4), "ms_per_launch": round(t_factor, 4),
                           "traffic": traffic_from_profiles("mq_factor_chol_grouped", C=C, G=1, panels=panels)},
        "mq_gptq_loop_chol": {"achieved": round(flop_loop / t_loop / 1e9, 2), "peak": PEAK_FP32_MFMA, "unit": "TFLOP/s",
                              "frac": round(flop_loop / t_loop / 1e9 / PEAK_FP32_MFMA, 4), "ms_per_launch": round(t_loop, 4),
                              "traffic": traffic_from_profiles("mq_gptq_loop_chol_grouped", C=C, R=R, G=1, batch=8)},
        "note": "a lone C = 7168 call is a chain of 55 dependent steps (one-workgroup diagonal blocks, 64-row column walks); "
                "the lone calls of the wide matrices (C = 16384, 18432) are in phases.other_configs",
    }

    cpu = None
    if not args.no_cpu_baseline:
        from oracle import gptq_oracle as O

        torch.set_num_threads(min(16, os.cpu_count() or 1))
        # the same linear again and again until about 10 s of CPU work are on the clock
        reps, t0 = 0, time.perf_counter()
        while reps == 0 or (time.perf_counter() - t0 < 10.0 and reps < 20):
            Hc, _ = O.hessian_update(None, 0, case.X)
            ref = O.quantize_linear(case.W, Hc)
            O.pack_weight({"qweight": ref["qweight"], "scale": ref["scale"], "zero": ref["zero"]}, 4, True, 128)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        cpu = {
            "value": round(1.0 / dt, 5),
            "unit": "linears/s",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"{reps} x one full config-1 linear ({R}x{C}, {n} tokens): torch CPU Hessian + 3-call Cholesky chain + "
                      f"column loop + pack, {dt:.1f} s each",
            "host_cpu_count": os.cpu_count(),
        }
        match = (out_q.cpu() == ref["qweight"]).float().mean().item()
        phases["code_match_vs_cpu_oracle"] = round(match, 6)
        phases["code_match_gate"] = 0.999
        phases["scales_equal_cpu_oracle"] = bool(torch.equal(out_s.cpu(), ref["scale"]))

    del H, Hd, A, F, Wt, Wt0, Qt, codes, X, Xsets, layers, outs, packed
    torch.cuda.empty_cache()
    with_cpu = not args.no_cpu_baseline
    if not args.no_other_configs and args.scale == 1.0:
        # the other configurations' linears, one at a time (their shapes have no sibling in a block to share grouped
        # calls with): wall per linear, the three big phases against their yardsticks, a roofline object each
        phases["other_configs"] = {
            "config2": config2_run(dev, with_cpu, reps=3),
            "config4": config4_run(dev, with_cpu, reps=2),
            "config5": config5_run(dev, with_cpu, reps=2, groups=(128, 32)),
        }
    # the third number of the headline metric: one pass over the whole MoE layer (config 3), outside the timed steps
    if not args.no_moe_layer and args.scale == 1.0:
        moe = moe_layer_run(args, with_cpu_oracle=with_cpu)
        phases["moe_layer_wall_s"] = moe["wall_s"]
        phases["moe_layer"] = moe
        # and once in the reference's order: every Hessian of the layer resident before the first linear is quantized
        args.no_overlap = True
        ref_order = moe_layer_run(args, with_cpu_oracle=False)
        phases["moe_layer_wall_s_all_hessians_resident_first"] = ref_order["wall_s"]
        phases["moe_layer_all_hessians_resident_first"] = {k: ref_order[k] for k in ("wall_s", "seconds",
                                                            "quantization_overlaps_hessian_collection")}

    line = {
        "metric": "GPTQ linears/sec (2048x7168 expert, g128)",
        "value": round(1000.0 / ms_per_step, 3),
        "unit": "linears/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "config 1: expert gate_proj 2048x7168 bf16, 8192 calibration tokens, 4-bit sym g128 B128; "
            "step = Hessian SYRK + factorisation + GPTQ loop + int32 packing",
            "R": R, "C": C, "tokens": n, "streams": n_lanes, "linears_per_grouped_call": group,
            "batches_of_the_timed_steps": batches(args.steps, n_lanes, group),
            "setup_linears_before_warmup": len(lanes) * max(prime) if prime else 0,
            "inputs": "every linear in flight has its own tokens and weights (streams x linears_per_grouped_call sets)",
        },
        "value_h_ready_to_packed": round(1000.0 / ms_h_ready, 3),
        "ms_per_step_h_ready_to_packed": round(ms_h_ready, 3),
        "ms_per_step_one_stream": round(ms_single, 3),
        "host_queueing_ms_per_step": round(host_issue_ms, 3),
        "roofline": roofline,
        "roofline_one_linear_per_call": roofline_lone,
        "cpu_baseline": cpu,
        "phases": phases,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
