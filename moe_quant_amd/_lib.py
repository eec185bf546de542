"""ctypes binding of libmoequant_hip.so.  There is no fallback: if the library is missing the
import of any kernel raises, and every wrapper refuses CPU tensors."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmoequant_hip.so")

MQ_OK, MQ_ERR_ARG, MQ_ERR_LAUNCH, MQ_ERR_WORKSPACE, MQ_ERR_TOO_LARGE = 0, -1, -2, -3, -4
DT_F32, DT_BF16, DT_F16 = 0, 1, 2

_vp, _i, _l, _f, _sz = C.c_void_p, C.c_int, C.c_long, C.c_float, C.c_size_t

# name -> (restype, argtypes); mirrors include/moequant_hip.h declaration by declaration
SIGNATURES = {
    "mq_hessian_syrk_workspace_bytes": (_sz, [_i, _i]),
    "mq_hessian_syrk": (_i, [_vp, _l, _vp, _i, _l, _i, _i, _f, _f, _i, _vp, _sz, _vp]),
    "mq_hessian_syrk_bf16": (_i, [_vp, _l, _vp, _l, _i, _i, _f, _f, _i, _vp, _sz, _vp]),
    "mq_hessian_syrk_grouped_workspace_bytes": (_sz, [_i, _vp, _i]),
    "mq_hessian_syrk_grouped": (_i, [_i, _vp, _vp, _vp, _i, _vp, _vp, _i, _vp, _vp, _i, _vp, _sz, _vp]),
    "mq_hessian_syrk_bf16_grouped": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _vp, _sz, _vp]),
    "mq_packed_tokens_bytes": (_sz, [_i, _i]),
    "mq_pack_tokens": (_i, [_vp, _i, _l, _vp, _i, _i, _vp, _vp, _l, _vp]),
    "mq_hessian_syrk_packed_workspace_bytes": (_sz, [_i, _i]),
    "mq_hessian_syrk_packed": (_i, [_vp, _l, _vp, _i, _i, _i, _f, _f, _i, _vp, _sz, _vp]),
    "mq_hessian_syrk_packed_grouped": (_i, [_i, _vp, _vp, _vp, _i, _vp, _i, _vp, _vp, _i, _vp]),
    "mq_symmetrize_upper": (_i, [_vp, _l, _i, _vp]),
    "mq_hessian_prestep": (_i, [_vp, _l, _i, _i, _vp, _vp, _vp]),
    "mq_permute_symmetric": (_i, [_vp, _l, _vp, _vp, _l, _i, _vp]),
    "mq_hessian_damp_workspace_bytes": (_sz, [_i]),
    "mq_hessian_damp": (_i, [_vp, _l, _i, _vp, _i, _l, _i, _vp, _f, _vp, _vp, _sz, _vp]),
    "mq_hessian_damp_noalloc": (_i, [_vp, _l, _i, _vp, _i, _l, _i, _vp, _f, _vp, _vp]),
    "mq_factor_upper_inverse": (_i, [_vp, _l, _i, _i, _vp, _vp]),
    "mq_factor_upper_inverse_from": (_i, [_vp, _l, _vp, _l, _i, _i, _vp, _vp]),
    "mq_factor_upper_inverse_grouped": (_i, [_i, _vp, _l, _vp, _l, _i, _i, _vp, _vp]),
    "mq_factor_chol_workspace_bytes": (_sz, [_i]),
    "mq_factor_chol": (_i, [_vp, _l, _vp, _l, _i, _vp, _vp, _sz, _vp]),
    "mq_factor_chol_grouped": (_i, [_i, _vp, _l, _vp, _l, _i, _vp, _vp, _sz, _vp]),
    "mq_quant_grid_sym": (_i, [_vp, _i, _l, _i, _i, _i, _i, _vp, _i, _vp, _vp, _vp]),
    "mq_mse_scale_sym": (_i, [_vp, _i, _l, _i, _i, _i, _vp, _vp, _i, _f, _f, _f, _i, _vp, _vp, _vp]),
    "mq_prepare_wt": (_i, [_vp, _i, _l, _i, _i, _vp, _vp, _vp, _l, _vp]),
    "mq_prepare_wt_pair": (_i, [_vp, _i, _l, _i, _i, _vp, _vp, _vp, _vp, _l, _vp]),
    "mq_gptq_loop_chol": (_i, [_vp, _vp, _l, _i, _i, _vp, _l, _vp, _l, _vp, _vp, _f, _f, _i, _i, _vp, _vp, _vp]),
    "mq_gptq_loop_chol_grouped": (_i, [_i, _vp, _vp, _l, _i, _i, _vp, _l, _vp, _l, _vp, _vp, _f, _f, _i, _i, _vp, _vp, _vp]),
    "mq_gptq_loop_scratch_bytes": (_sz, [_i]),
    "mq_gptq_loop": (_i, [_vp, _l, _i, _i, _vp, _l, _vp, _l, _vp, _vp, _f, _f, _i, _i, _vp, _vp, _vp]),
    "mq_gptq_loop_grouped": (_i, [_i, _vp, _l, _i, _i, _vp, _l, _vp, _l, _vp, _vp, _f, _f, _i, _i, _vp, _vp, _vp]),
    "mq_untranspose_codes": (_i, [_vp, _i, _i, _vp, _vp, _l, _vp]),
    "mq_pack_int4": (_i, [_vp, _l, _i, _i, _vp, _i, _vp, _l, _vp]),
    "mq_pack_from_qt": (_i, [_vp, _i, _i, _vp, _vp, _l, _vp]),
    "mq_dequant_fp8_block": (_i, [_vp, _l, _i, _i, _vp, _l, _i, _vp, _l, _vp]),
    "mq_swiglu": (_i, [_vp, _l, _i, _i, _i, _vp, _l, _vp]),
    "mq_swiglu_packed": (_i, [_vp, _l, _vp, _l, _i, _i, _i, _vp, _vp]),
    "mq_gemm_f32": (_i, [_vp, _l, _l, _vp, _l, _l, _vp, _l, _i, _i, _i, _f, _f, _i, _i, _vp]),
}

_lib = None


class MoeQuantHipError(RuntimeError):
    pass


def load():
    """Load the shared library (once) and attach signatures."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise MoeQuantHipError(
            f"{LIB_PATH} is missing: the HIP kernels are not built. Run `python -m moe_quant_amd.build` "
            "(needs hipcc). There is no CPU or torch fallback for this engine."
        )
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


_ERR = {MQ_ERR_ARG: "bad argument", MQ_ERR_LAUNCH: "kernel launch failed", MQ_ERR_WORKSPACE: "workspace too small",
        MQ_ERR_TOO_LARGE: "problem larger than the entry point's fixed scratch capacity"}


def check(rc: int, what: str) -> None:
    if rc != MQ_OK:
        raise MoeQuantHipError(f"{what} failed: {_ERR.get(rc, rc)} (code {rc})")
