"""Drop-in for MoE-Quant's src/linalg_utils.py, computed by the HIP factorisation kernels."""
from __future__ import annotations

import torch
from torch import Tensor

from . import ops

__all__ = ["inv_sym", "inverse_cholesky_factor"]


def _padded_copy(X: Tensor) -> Tensor:
    """fp32 copy of X padded with an identity block to a multiple of 128 (diag(X, I) factors to diag(U, I))."""
    C = X.shape[0]
    Cp = (C + 127) // 128 * 128
    if Cp == C:
        return X.to(torch.float32, copy=True).contiguous()
    A = torch.zeros(Cp, Cp, dtype=torch.float32, device=X.device)
    A[:C, :C] = X
    A.diagonal()[C:] = 1.0
    return A


def inverse_cholesky_factor(H: Tensor, normalize: bool = True):
    """Upper U = chol(H^-1, upper), rows divided by the diagonal when `normalize` (what
    GPTQ._get_hessian_inverse returns, src/gptq.py:236-242).  H is not modified.
    Returns (U, info): info is a device int32 tensor, 0 on success, else the 1-based pivot that failed."""
    C = H.shape[0]
    if (C % 128 == 0 and H.dtype == torch.float32 and H.stride(1) == 1 and H.stride(0) % 4 == 0
            and H.data_ptr() % 16 == 0):
        return ops.factor_upper_inverse_from(H, normalize=normalize)  # reads H in place of a copy of it
    A = _padded_copy(H)
    info = ops.factor_upper_inverse_(A, normalize=normalize)
    U = A if A.shape[0] == C else A[:C, :C].contiguous()
    return U, info


def inv_sym(X: Tensor) -> Tensor:
    """X^-1 for symmetric positive definite X (src/linalg_utils.py:8-12), assembled as R^-T R^-1 from the
    same factor the GPTQ path uses.  Raises torch.linalg.LinAlgError when X is not positive definite,
    as torch.linalg.cholesky does."""
    C = X.shape[0]
    A = _padded_copy(X)
    info = int(ops.factor_upper_inverse_(A, normalize=False).item())
    if info != 0:
        raise torch.linalg.LinAlgError(f"inv_sym: the matrix is not positive definite (pivot {info})")
    Cp = A.shape[0]
    out = torch.empty(Cp, Cp, dtype=torch.float32, device=X.device)
    # out[m,n] = sum_k Rinv[k,m] Rinv[k,n]
    ops.gemm_f32_(A, 1, Cp, A, Cp, 1, out, Cp, Cp, Cp)
    return out if Cp == C else out[:C, :C].contiguous()
