"""CPU-side checks: the C-ABI library loads and exports what include/moequant_hip.h declares, the
ctypes table matches the header, and the host mirror keeps the reference's API surface."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "moequant_hip.h")


def _declared():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    decls = {}
    for m in re.finditer(r"\b(int|size_t)\s+(mq_\w+)\s*\(([^;]*?)\)\s*;", src, flags=re.S):
        args = [a.strip() for a in m.group(3).split(",")]
        decls[m.group(2)] = (m.group(1), args)
    return decls


def test_header_declares_the_expected_entry_points():
    d = _declared()
    for name in ("mq_hessian_syrk", "mq_hessian_syrk_grouped", "mq_hessian_syrk_bf16", "mq_factor_upper_inverse", "mq_quant_grid_sym", "mq_prepare_wt",
                 "mq_gptq_loop", "mq_untranspose_codes", "mq_pack_int4", "mq_pack_from_qt", "mq_gemm_f32",
                 "mq_hessian_syrk_workspace_bytes"):
        assert name in d


def test_library_exports_every_declared_symbol():
    from moe_quant_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail(f"{_lib.LIB_PATH} missing: run `python -m moe_quant_amd.build`")
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"


def test_ctypes_table_matches_header_arity():
    from moe_quant_amd import _lib

    d = _declared()
    assert set(d) == set(_lib.SIGNATURES), set(d) ^ set(_lib.SIGNATURES)
    for name, (ret, args) in d.items():
        res, argtypes = _lib.SIGNATURES[name]
        assert len(argtypes) == len(args), name
        assert (res is ctypes.c_size_t) == (ret == "size_t"), name
        for a, t in zip(args, argtypes):
            if "*" in a:
                assert t is ctypes.c_void_p, (name, a)
            elif a.startswith("long"):
                assert t is ctypes.c_long, (name, a)
            elif a.startswith("float"):
                assert t is ctypes.c_float, (name, a)
            elif a.startswith("size_t"):
                assert t is ctypes.c_size_t, (name, a)
            else:
                assert t is ctypes.c_int, (name, a)
    _lib.load()  # attaches every signature; raises on a missing symbol


def test_pure_size_query_needs_no_gpu():
    from moe_quant_amd import _lib

    lib = _lib.load()
    # wide and long: the tokens are re-laid out into the workspace first (8192 x 7168 16-bit values, no padding needed)
    assert lib.mq_hessian_syrk_workspace_bytes(8192, 7168) == lib.mq_packed_tokens_bytes(8192, 7168) == 8192 * 7168 * 2
    assert lib.mq_packed_tokens_bytes(100, 264) == 128 * 512 * 2  # tokens padded to 128, channels to 256
    assert lib.mq_hessian_syrk_workspace_bytes(2048, 7168) == 0  # enough tiles to fill the GPU, too short to re-lay out
    need = lib.mq_hessian_syrk_workspace_bytes(65536, 2048)  # 36 tiles of 256x256: the token range is split
    assert need > 0 and need % (36 * 256 * 256 * 4) == 0
    assert lib.mq_hessian_syrk_workspace_bytes(0, 128) == 0


def test_no_cpu_path():
    from moe_quant_amd import _lib, ops
    from moe_quant_amd.linalg_utils import inv_sym

    with pytest.raises(_lib.MoeQuantHipError):
        ops.pack_int4(torch.zeros(2, 8, dtype=torch.uint8))
    with pytest.raises(_lib.MoeQuantHipError):
        inv_sym(torch.eye(128))
    with pytest.raises(_lib.MoeQuantHipError):
        ops.hessian_syrk_(torch.zeros(128, 128), torch.zeros(4, 128, dtype=torch.bfloat16), 0.0, 1.0)


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "moe_quant_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")):
                txt = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in txt, os.path.join(dirpath, f)


def test_handle_surface_matches_reference():
    from moe_quant_amd.gptq import GPTQ, QuantizationOrder

    lin = torch.nn.Linear(256, 64, bias=False, dtype=torch.bfloat16)
    h = GPTQ(lin, group_size=128, sym=True, rel_damp=0.01, block_size=128, quantization_order="activation",
             quantization_scale="absmax", is_distributed=False, tied_gptq_handle=None)
    assert (h.d_row, h.d_col) == (64, 256) and h.block_size == 128 and h.H is None and h.num_samples == 0
    assert h.quantization_order is QuantizationOrder.ACTIVATION and h.tokens_collected == 0
    assert h.W is lin.weight and h.W_dtype == torch.bfloat16 and h.W_shape == lin.weight.shape
    assert not h.has_hessian_issues() and GPTQ.add_batch is GPTQ.update
    for attr in ("quantize", "quantization_pre_step", "_quantize", "_get_hessian_inverse", "reset", "update"):
        assert callable(getattr(h, attr))
    assert GPTQ(lin).block_size == 256  # `block_size or d_col`
    with pytest.raises(AssertionError):
        GPTQ(torch.nn.Conv2d(3, 3, 1))
    with pytest.raises(ValueError):
        GPTQ(lin, quantization_order="nonsense")
    # tie bookkeeping: src/gptq.py:56-59,113-118
    owner = GPTQ(lin, 128, True)
    tied = GPTQ(lin, 128, True, tied_gptq_handle=owner)
    assert owner.num_tied_handles == 1
    owner.H = torch.eye(256)
    owner.reset()
    assert owner.H is not None  # still needed by the tied handle
    tied.H = owner.H
    tied.reset()
    # as in the reference, a tied handle (which itself has no dependants) takes the first branch of
    # reset(): it drops its own reference and never decrements the owner's counter
    assert tied.H is None and owner.num_tied_handles == 1 and owner.H is not None
    with pytest.raises(TypeError):
        h.update(torch.zeros(4, 256, dtype=torch.float64))  # only the reference driver's dtypes: fp16, bf16, fp32
    h.update(torch.zeros(0, 256))  # an empty batch is a no-op (and touches no kernel)
    assert h.H is None and h.tokens_collected == 0


def test_reference_module_names_resolve():
    import moe_quant_amd as m

    assert callable(m.gptq_loop.gptq_loop) and callable(m.linalg_utils.inv_sym)
    assert callable(m.quant_utils.get_quantization_grid) and callable(m.quant_utils.dequantize_linear_weight)
    assert callable(m.quant_utils.get_relative_mse_error) and callable(m.pack_quantized_model.pack_weight)
    # torch helpers that stay torch: same results as the oracle's restatement
    from oracle import gptq_oracle as O

    q = torch.randint(0, 16, (4, 32), dtype=torch.uint8)
    s = torch.rand(4, 2).bfloat16() * 0.01 + 0.001
    z = torch.full((4, 2), 8.0).bfloat16()
    assert torch.equal(m.quant_utils.dequantize_linear_weight(q, s, z), O.dequantize_linear_weight(q, s, z))
    w = torch.randn(4, 32)
    assert torch.equal(m.quant_utils.get_relative_mse_error(w * 0.9, w), O.relative_mse(w * 0.9, w))


def test_prepare_quantization_config_takes_the_reference_namespace():
    """pack_quantized_model.py:78 passes its argparse namespace; the three values give the same dict."""
    import argparse

    from moe_quant_amd.pack_quantized_model import prepare_quantization_config

    ns = argparse.Namespace(bits=4, group_size=128, quantize_only_experts=True, other="ignored")
    a, b = prepare_quantization_config(ns), prepare_quantization_config(4, 128, True)
    assert a == b and a["config_groups"]["group_0"]["weights"]["group_size"] == 128 and len(a["ignore"]) == 4
    assert prepare_quantization_config(argparse.Namespace(bits=4, group_size=64, quantize_only_experts=False))["ignore"] == ["lm_head"]
