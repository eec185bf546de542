"""Tensor-level wrappers over the C ABI.  torch is used for device memory and the current stream only;
every computation below happens in libmoequant_hip.so."""
from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor

from . import _lib
from ._lib import DT_BF16, DT_F16, DT_F32, check

_DT = {torch.float32: DT_F32, torch.bfloat16: DT_BF16, torch.float16: DT_F16}


def _dt(dtype: Optional[torch.dtype]) -> int:
    if dtype is None:
        return DT_F32
    if dtype not in _DT:
        raise TypeError(f"unsupported dtype {dtype}")
    return _DT[dtype]


def _stream(t: Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _dev(*ts: Optional[Tensor]) -> None:
    for t in ts:
        if t is not None and not t.is_cuda:
            raise _lib.MoeQuantHipError("moe_quant_amd kernels need GPU tensors; there is no CPU path")


def _p(t: Optional[Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


class _Workspace:
    """One growing scratch buffer per (device, stream, purpose), so the hot path does not hit the allocator and
    linears queued on different streams never share scratch memory."""

    def __init__(self):
        self.buf = {}

    def get(self, device: torch.device, nbytes: int, purpose: str = "") -> Tensor:
        key = (device.type, device.index, torch.cuda.current_stream(device).cuda_stream, purpose)
        b = self.buf.get(key)
        if b is None or b.numel() < nbytes:
            b = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
            self.buf[key] = b
        return b


_ws = _Workspace()


# ---- (1) Hessian ------------------------------------------------------------------------------------
def hessian_syrk_(H: Tensor, X: Tensor, beta: float, alpha: float, mirror: bool = True) -> Tensor:
    """H <- beta*H + alpha*X^T X in place.  H (C,C) fp32, X (n,C) bf16, fp16 or fp32, rows may be strided."""
    _dev(H, X)
    lib = _lib.load()
    C = H.shape[0]
    if H.dtype != torch.float32 or H.shape != (C, C) or H.stride(1) != 1:
        raise ValueError("H must be a (C,C) fp32 matrix with unit column stride")
    if X.dtype not in _DT or X.dim() != 2 or X.shape[1] != C:
        raise ValueError("X must be (n,C) bf16, fp16 or fp32")
    if X.shape[0] > 0 and X.stride(1) != 1:
        X = X.contiguous()
    n = X.shape[0]
    need = lib.mq_hessian_syrk_workspace_bytes(n, C) if X.dtype != torch.float32 else 0
    ws = _ws.get(H.device, need, "syrk") if need else None
    ldx = X.stride(0) if n > 1 else C
    rc = lib.mq_hessian_syrk(
        H.data_ptr(), H.stride(0), X.data_ptr() if n else None, _DT[X.dtype], ldx, n, C, beta, alpha, int(mirror),
        _p(ws), need, _stream(H),
    )
    check(rc, "mq_hessian_syrk")
    return H


def hessian_syrk_grouped_(Hs, Xs, betas, alphas, mirror: bool = True) -> None:
    """H_i <- beta_i*H_i + alpha_i*X_i^T X_i for several Hessians of one width in one call (lists of equal length)."""
    import ctypes as C_

    lib = _lib.load()
    k = len(Hs)
    if not (len(Xs) == len(betas) == len(alphas) == k):
        raise ValueError("Hs, Xs, betas, alphas must have the same length")
    if k == 0:
        return
    _dev(*Hs, *Xs)
    C = Hs[0].shape[0]
    Xs = [x if (x.shape[0] == 0 or x.stride(1) == 1) else x.contiguous() for x in Xs]
    xdt = Xs[0].dtype
    for H, X in zip(Hs, Xs):
        if H.dtype != torch.float32 or H.shape != (C, C) or H.stride(1) != 1:
            raise ValueError("every H must be a (C,C) fp32 matrix with unit column stride")
        if X.dtype not in _DT or X.dtype != xdt or X.dim() != 2 or X.shape[1] != C:
            raise ValueError("every X must be (n,C), all of one type (bf16, fp16 or fp32)")
    ns = (C_.c_int * k)(*[x.shape[0] for x in Xs])
    Hp = (C_.c_void_p * k)(*[h.data_ptr() for h in Hs])
    Xp = (C_.c_void_p * k)(*[(x.data_ptr() if x.shape[0] else None) for x in Xs])
    ldh = (C_.c_long * k)(*[h.stride(0) for h in Hs])
    ldx = (C_.c_long * k)(*[(x.stride(0) if x.shape[0] > 1 else C) for x in Xs])
    be = (C_.c_float * k)(*[float(b) for b in betas])
    al = (C_.c_float * k)(*[float(a) for a in alphas])
    need = lib.mq_hessian_syrk_grouped_workspace_bytes(k, ns, C)
    ws = _ws.get(Hs[0].device, need, "syrk") if need else None
    rc = lib.mq_hessian_syrk_grouped(k, Hp, ldh, Xp, _DT[xdt], ldx, ns, C, be, al, int(mirror), _p(ws), need,
                                     _stream(Hs[0]))
    check(rc, "mq_hessian_syrk_grouped")


class PackedTokens:
    """Activations laid out for the matrix cores: Xp[o][c][j] = X[8 o + j][c] (token octet o, channel c padded to a
    multiple of 256, j = 0..7), tokens padded with zeros to a multiple of 32.  Made by `pack_tokens`, read by
    `hessian_syrk_packed_`."""

    def __init__(self, data: Tensor, n: int, C: int, dtype: torch.dtype):
        self.data, self.n, self.C, self.dtype = data, n, C, dtype


def pack_tokens(X: Tensor, rows: Optional[Tensor] = None, also_token_major: bool = False):
    """X (m, C) bf16/fp16 -> PackedTokens of X (rows None) or of X[rows] (rows: int64 indices on the device; the
    gather and the re-layout are one pass).  also_token_major: returns (PackedTokens, Xg) with Xg the gathered rows
    once more as an ordinary (n, C) tensor, written by the same pass (for the GEMMs of the model's forward)."""
    _dev(X, rows)
    lib = _lib.load()
    if X.dim() != 2 or X.dtype not in (torch.bfloat16, torch.float16) or X.stride(1) != 1:
        raise ValueError("X must be (m, C) bf16/fp16 with unit column stride")
    if rows is not None and (rows.dtype != torch.int64 or rows.dim() != 1 or not rows.is_contiguous()):
        raise ValueError("rows must be a contiguous int64 vector")
    C = X.shape[1]
    n = X.shape[0] if rows is None else rows.numel()
    nbytes = lib.mq_packed_tokens_bytes(n, C)
    out = torch.empty(max(nbytes, 16) // 2, dtype=X.dtype, device=X.device)
    Xg = torch.empty(n, C, dtype=X.dtype, device=X.device) if also_token_major else None
    rc = lib.mq_pack_tokens(X.data_ptr(), _DT[X.dtype], X.stride(0), _p(rows), n, C, out.data_ptr(), _p(Xg), C, _stream(X))
    check(rc, "mq_pack_tokens")
    P = PackedTokens(out, n, C, X.dtype)
    return (P, Xg) if also_token_major else P


def unpack_tokens(P: PackedTokens) -> Tensor:
    """PackedTokens -> the ordinary (n, C) tensor (a torch view/copy; for tests and debugging)."""
    Cp = (P.C + 255) // 256 * 256
    octets = (P.n + 127) // 128 * 16
    return P.data[: octets * Cp * 8].view(octets, Cp, 8).permute(0, 2, 1).reshape(octets * 8, Cp)[: P.n, : P.C].contiguous()


def hessian_syrk_packed_(H: Tensor, Xp: PackedTokens, beta: float, alpha: float, mirror: bool = True) -> Tensor:
    """H <- beta*H + alpha*X^T X in place, X given as PackedTokens."""
    _dev(H, Xp.data)
    lib = _lib.load()
    C = H.shape[0]
    if H.dtype != torch.float32 or H.shape != (C, C) or H.stride(1) != 1 or Xp.C != C:
        raise ValueError("H must be a (C,C) fp32 matrix with unit column stride, C the packed tokens' width")
    if Xp.n <= 0:
        if beta != 1.0:
            H.mul_(beta)
        return H
    need = lib.mq_hessian_syrk_packed_workspace_bytes(Xp.n, C)
    ws = _ws.get(H.device, need, "syrk") if need else None
    rc = lib.mq_hessian_syrk_packed(H.data_ptr(), H.stride(0), Xp.data.data_ptr(), _DT[Xp.dtype], Xp.n, C, beta, alpha,
                                    int(mirror), _p(ws), need, _stream(H))
    check(rc, "mq_hessian_syrk_packed")
    return H


def hessian_syrk_packed_grouped_(Hs, Xps, betas, alphas, mirror: bool = True) -> None:
    """hessian_syrk_packed_ for several Hessians of one width with one library call (every problem at least one token)."""
    import ctypes as C_

    lib = _lib.load()
    k = len(Hs)
    if not (len(Xps) == len(betas) == len(alphas) == k):
        raise ValueError("Hs, Xps, betas, alphas must have the same length")
    if k == 0:
        return
    _dev(*Hs, *[x.data for x in Xps])
    C = Hs[0].shape[0]
    dt = Xps[0].dtype
    for H, X in zip(Hs, Xps):
        if H.dtype != torch.float32 or H.shape != (C, C) or H.stride(1) != 1:
            raise ValueError("every H must be a (C,C) fp32 matrix with unit column stride")
        if X.C != C or X.dtype != dt or X.n <= 0:
            raise ValueError("every packed X must have C channels, one dtype and at least one token")
    ns = (C_.c_int * k)(*[x.n for x in Xps])
    Hp = (C_.c_void_p * k)(*[h.data_ptr() for h in Hs])
    Xp = (C_.c_void_p * k)(*[x.data.data_ptr() for x in Xps])
    ldh = (C_.c_long * k)(*[h.stride(0) for h in Hs])
    be = (C_.c_float * k)(*[float(b) for b in betas])
    al = (C_.c_float * k)(*[float(a) for a in alphas])
    rc = lib.mq_hessian_syrk_packed_grouped(k, Hp, ldh, Xp, _DT[dt], ns, C, be, al, int(mirror), _stream(Hs[0]))
    check(rc, "mq_hessian_syrk_packed_grouped")


def symmetrize_upper_(H: Tensor) -> Tensor:
    """Copies the upper triangle of H onto the lower one, in place."""
    _dev(H)
    lib = _lib.load()
    C = H.shape[0]
    if H.dtype != torch.float32 or H.shape != (C, C) or H.stride(1) != 1:
        raise ValueError("H must be a (C,C) fp32 matrix with unit column stride")
    check(lib.mq_symmetrize_upper(H.data_ptr(), H.stride(0), C, _stream(H)), "mq_symmetrize_upper")
    return H


def hessian_prestep_(H: Tensor, upper_only: bool) -> Tuple[Tensor, Tensor]:
    """In place: mirror the upper triangle (when `upper_only`), NaN -> identity, zero diagonal entries -> 1.
    Returns (pruned (C,) uint8, flags (4,) int32), both on the device; nothing is read back."""
    _dev(H)
    lib = _lib.load()
    C = H.shape[0]
    if H.dtype != torch.float32 or H.shape != (C, C) or H.stride(1) != 1:
        raise ValueError("H must be a (C,C) fp32 matrix with unit column stride")
    pruned = torch.empty(C, dtype=torch.uint8, device=H.device)
    flags = torch.empty(4, dtype=torch.int32, device=H.device)
    rc = lib.mq_hessian_prestep(H.data_ptr(), H.stride(0), C, int(upper_only), pruned.data_ptr(), flags.data_ptr(),
                                _stream(H))
    check(rc, "mq_hessian_prestep")
    return pruned, flags


def permute_symmetric(H: Tensor, perm: Tensor) -> Tensor:
    """H[perm][:, perm] as a new tensor, in one pass (perm: int32 of length C on the device)."""
    _dev(H, perm)
    lib = _lib.load()
    C = H.shape[0]
    if H.dtype != torch.float32 or H.shape != (C, C) or H.stride(1) != 1:
        raise ValueError("H must be a (C,C) fp32 matrix with unit column stride")
    if perm.dtype != torch.int32 or perm.numel() != C or not perm.is_contiguous():
        raise ValueError("perm must be a contiguous int32 vector of length C")
    Hp = torch.empty((C, C), dtype=torch.float32, device=H.device)
    check(lib.mq_permute_symmetric(H.data_ptr(), H.stride(0), perm.data_ptr(), Hp.data_ptr(), C, C, _stream(H)),
          "mq_permute_symmetric")
    return Hp


def hessian_damp_(H: Tensor, W: Tensor, pruned: Optional[Tensor], rel_damp: float, flags: Tensor) -> Tensor:
    """In place: rows/columns of H for all-zero (or pruned) weight columns cleared with a unit diagonal, then
    rel_damp * mean(diag) added to the diagonal."""
    _dev(H, W, pruned, flags)
    lib = _lib.load()
    C = H.shape[0]
    if H.dtype != torch.float32 or H.shape != (C, C) or H.stride(1) != 1:
        raise ValueError("H must be a (C,C) fp32 matrix with unit column stride")
    if W.dim() != 2 or W.shape[1] != C:
        raise ValueError("W must be (R,C)")
    if W.stride(1) != 1:
        W = W.contiguous()
    need = lib.mq_hessian_damp_workspace_bytes(C)
    ws = _ws.get(H.device, need, "damp")
    rc = lib.mq_hessian_damp(H.data_ptr(), H.stride(0), C, W.data_ptr(), _dt(W.dtype), W.stride(0), W.shape[0],
                             _p(pruned), float(rel_damp), flags.data_ptr(), ws.data_ptr(), need, _stream(H))
    check(rc, "mq_hessian_damp")
    return H


def hessian_damp_noalloc_(H: Tensor, W: Tensor, pruned: Optional[Tensor], rel_damp: float, flags: Tensor) -> Tensor:
    """hessian_damp_ through the entry point that brings its own scratch memory: allocates nothing (neither here
    nor in the library), C <= 32768, calls on one GPU must not overlap."""
    _dev(H, W, pruned, flags)
    lib = _lib.load()
    C = H.shape[0]
    if H.dtype != torch.float32 or H.shape != (C, C) or H.stride(1) != 1:
        raise ValueError("H must be a (C,C) fp32 matrix with unit column stride")
    if W.dim() != 2 or W.shape[1] != C or W.stride(1) != 1:
        raise ValueError("W must be (R,C) with unit column stride")
    rc = lib.mq_hessian_damp_noalloc(H.data_ptr(), H.stride(0), C, W.data_ptr(), _dt(W.dtype), W.stride(0), W.shape[0],
                                     _p(pruned), float(rel_damp), flags.data_ptr(), _stream(H))
    check(rc, "mq_hessian_damp_noalloc")
    return H


# ---- (2) factorisation -------------------------------------------------------------------------------
def factor_upper_inverse_(A: Tensor, info: Optional[Tensor] = None, normalize: bool = True) -> Tensor:
    """In place A -> upper U = chol(A^-1, upper), rows scaled to unit diagonal when `normalize`.
    Returns the device int32 `info` (0 = success)."""
    _dev(A, info)
    lib = _lib.load()
    C = A.shape[0]
    if A.dtype != torch.float32 or A.shape != (C, C) or A.stride(1) != 1 or C % 128:
        raise ValueError("A must be (C,C) fp32, unit column stride, C % 128 == 0")
    if info is None:
        info = torch.zeros(1, dtype=torch.int32, device=A.device)
    rc = lib.mq_factor_upper_inverse(A.data_ptr(), A.stride(0), C, int(normalize), info.data_ptr(), _stream(A))
    check(rc, "mq_factor_upper_inverse")
    return info


def factor_upper_inverse_from(H: Tensor, info: Optional[Tensor] = None, normalize: bool = True):
    """Like factor_upper_inverse_ but H is left untouched: returns (U, info) with U a new tensor."""
    _dev(H, info)
    lib = _lib.load()
    C = H.shape[0]
    if H.dtype != torch.float32 or H.shape != (C, C) or H.stride(1) != 1 or C % 128:
        raise ValueError("H must be (C,C) fp32, unit column stride, C % 128 == 0")
    if info is None:
        info = torch.zeros(1, dtype=torch.int32, device=H.device)
    U = torch.empty((C, C), dtype=torch.float32, device=H.device)
    rc = lib.mq_factor_upper_inverse_from(H.data_ptr(), H.stride(0), U.data_ptr(), U.stride(0), C, int(normalize),
                                          info.data_ptr(), _stream(H))
    check(rc, "mq_factor_upper_inverse_from")
    return U, info


def _ptr_array(tensors):
    import ctypes as C_

    return (C_.c_void_p * len(tensors))(*[None if t is None else t.data_ptr() for t in tensors])


def factor_upper_inverse_from_grouped(Hs, normalize: bool = True):
    """factor_upper_inverse_from for several matrices of one size with one library call: returns (Us, infos), infos a
    device int32 vector with one word per matrix.  Bit-identical to separate calls."""
    _dev(*Hs)
    lib = _lib.load()
    k = len(Hs)
    if k == 0:
        return [], None
    C = Hs[0].shape[0]
    ld = Hs[0].stride(0)
    for H in Hs:
        if H.dtype != torch.float32 or H.shape != (C, C) or H.stride(1) != 1 or C % 128 or H.stride(0) != ld:
            raise ValueError("every H must be (C,C) fp32 with unit column stride, one pitch, C % 128 == 0")
    infos = torch.zeros(k, dtype=torch.int32, device=Hs[0].device)
    Us = [torch.empty((C, C), dtype=torch.float32, device=Hs[0].device) for _ in range(k)]
    import ctypes as C_

    ip = (C_.c_void_p * k)(*[infos.data_ptr() + 4 * i for i in range(k)])
    rc = lib.mq_factor_upper_inverse_grouped(k, _ptr_array(Hs), ld, _ptr_array(Us), C, C, int(normalize), ip, _stream(Hs[0]))
    check(rc, "mq_factor_upper_inverse_grouped")
    return Us, infos


def factor_chol_grouped(Hs):
    """Cholesky-only factorisation of several matrices of one size with one library call: returns (Fs, infos) with
    F[j,k] = -R[j,k]/R[k,k] above the diagonal (H = R R^T), the multipliers of gptq_loop_chol_; the diagonal and
    the lower triangle of every F are undefined.  Bit-identical to separate calls."""
    _dev(*Hs)
    lib = _lib.load()
    k = len(Hs)
    if k == 0:
        return [], None
    C = Hs[0].shape[0]
    ld = Hs[0].stride(0)
    for H in Hs:
        if H.dtype != torch.float32 or H.shape != (C, C) or H.stride(1) != 1 or C % 128 or H.stride(0) != ld:
            raise ValueError("every H must be (C,C) fp32 with unit column stride, one pitch, C % 128 == 0")
    dev = Hs[0].device
    infos = torch.zeros(k, dtype=torch.int32, device=dev)
    Fs = [torch.empty((C, C), dtype=torch.float32, device=dev) for _ in range(k)]
    need = lib.mq_factor_chol_workspace_bytes(C)
    ws = _ws.get(dev, need * k, "chol")
    import ctypes as C_

    ip = (C_.c_void_p * k)(*[infos.data_ptr() + 4 * i for i in range(k)])
    wp = (C_.c_void_p * k)(*[ws.data_ptr() + need * i for i in range(k)])
    rc = lib.mq_factor_chol_grouped(k, _ptr_array(Hs), ld, _ptr_array(Fs), C, C, ip, wp, need, _stream(Hs[0]))
    check(rc, "mq_factor_chol_grouped")
    return Fs, infos


def factor_chol(H: Tensor):
    """(F, info) for one matrix, see factor_chol_grouped."""
    Fs, infos = factor_chol_grouped([H])
    return Fs[0], infos


# ---- (3) grid, layout, loop --------------------------------------------------------------------------
def quant_grid_sym(W: Tensor, group_size: int, bits: int, round_dtype, dead_cols: Optional[Tensor] = None,
                   want_transposed: bool = True) -> Tuple[Tensor, Optional[Tensor]]:
    _dev(W, dead_cols)
    lib = _lib.load()
    R, C = W.shape
    if W.stride(1) != 1:
        W = W.contiguous()
    G = C // group_size
    s_rg = torch.empty(R, G, dtype=torch.float32, device=W.device)
    s_gr = torch.empty(G, R, dtype=torch.float32, device=W.device) if want_transposed else None
    rc = lib.mq_quant_grid_sym(W.data_ptr(), _dt(W.dtype), W.stride(0), R, C, group_size, bits, _p(dead_cols),
                               _dt(round_dtype), s_rg.data_ptr(), _p(s_gr), _stream(W))
    check(rc, "mq_quant_grid_sym")
    return s_rg, s_gr


def mse_scale_sym_(W: Tensor, group_size: int, p: Tensor, scale_rg: Tensor, scale_gr: Optional[Tensor], qzero: float,
                   maxq: float, norm: float, round_dtype, dead_cols: Optional[Tensor] = None) -> Tensor:
    """In place on scale_rg (R,G) fp32 (and its transposed copy scale_gr): the scale search over shrink factors p."""
    _dev(W, p, scale_rg, scale_gr, dead_cols)
    lib = _lib.load()
    R, C = W.shape
    if W.stride(1) != 1:
        W = W.contiguous()
    G = C // group_size
    if scale_rg.dtype != torch.float32 or scale_rg.shape != (R, G) or not scale_rg.is_contiguous():
        raise ValueError("scale_rg must be a contiguous (R,G) fp32 tensor")
    if scale_gr is not None and (scale_gr.dtype != torch.float32 or scale_gr.shape != (G, R) or not scale_gr.is_contiguous()):
        raise ValueError("scale_gr must be a contiguous (G,R) fp32 tensor")
    if p.dtype != torch.float32 or p.dim() != 1 or not p.is_contiguous():
        raise ValueError("p must be a contiguous fp32 vector")
    rc = lib.mq_mse_scale_sym(W.data_ptr(), _dt(W.dtype), W.stride(0), R, C, group_size, _p(dead_cols), p.data_ptr(),
                              p.numel(), float(qzero), float(maxq), float(norm), _dt(round_dtype), scale_rg.data_ptr(),
                              _p(scale_gr), _stream(W))
    check(rc, "mq_mse_scale_sym")
    return scale_rg


def prepare_wt(W: Tensor, perm: Optional[Tensor] = None, dead_cols: Optional[Tensor] = None) -> Tensor:
    _dev(W, perm, dead_cols)
    lib = _lib.load()
    R, C = W.shape
    if W.stride(1) != 1:
        W = W.contiguous()
    Wt = torch.empty(C, R, dtype=torch.float32, device=W.device)
    rc = lib.mq_prepare_wt(W.data_ptr(), _dt(W.dtype), W.stride(0), R, C, _p(perm), _p(dead_cols), Wt.data_ptr(), R,
                           _stream(W))
    check(rc, "mq_prepare_wt")
    return Wt


def prepare_wt_pair(W: Tensor, perm: Optional[Tensor] = None, dead_cols: Optional[Tensor] = None):
    """prepare_wt twice: (Wt, W0t), the copy the loop updates in place and the copy it keeps reading."""
    _dev(W, perm, dead_cols)
    lib = _lib.load()
    R, C = W.shape
    if W.stride(1) != 1:
        W = W.contiguous()
    Wt = torch.empty(C, R, dtype=torch.float32, device=W.device)
    W0t = torch.empty(C, R, dtype=torch.float32, device=W.device)
    rc = lib.mq_prepare_wt_pair(W.data_ptr(), _dt(W.dtype), W.stride(0), R, C, _p(perm), _p(dead_cols), Wt.data_ptr(),
                                W0t.data_ptr(), R, _stream(W))
    check(rc, "mq_prepare_wt_pair")
    return Wt, W0t


def gptq_loop_chol_grouped_(Wts, W0ts, Fs, scales, scale_rows, qzero_const: float, maxq: float, round_dtype, block: int):
    """The inverse-free loop for several linears of one shape with one library call: Fs from factor_chol_grouped,
    (Wts, W0ts) from prepare_wt_pair.  In place on every Wt; returns the list of code tensors Qt (C,R) uint8."""
    k = len(Wts)
    if not (len(W0ts) == len(Fs) == len(scales) == k) or (scale_rows is not None and len(scale_rows) != k):
        raise ValueError("Wts, W0ts, Fs, scales, scale_rows must have the same length")
    if k == 0:
        return []
    _dev(*Wts, *W0ts, *Fs, *scales, *(scale_rows or []))
    lib = _lib.load()
    C, R = Wts[0].shape
    ldw, ldf, lds = Wts[0].stride(0), Fs[0].stride(0), scales[0].stride(0)
    for Wt, W0t, F, sc in zip(Wts, W0ts, Fs, scales):
        for t in (Wt, W0t, F, sc):
            if t.dtype != torch.float32 or t.stride(-1) != 1:
                raise ValueError("Wt, W0t, F, scale must be fp32 with unit inner stride")
        if (Wt.shape != (C, R) or W0t.shape != (C, R) or Wt.stride(0) != ldw or W0t.stride(0) != ldw or F.stride(0) != ldf
                or sc.stride(0) != lds):
            raise ValueError("all linears of a group share one shape and one set of pitches")
    if scale_rows is not None:
        for m in scale_rows:
            if m.dtype != torch.int32 or m.numel() != C:
                raise ValueError("scale_row must be int32 of length C")
    elif scales[0].shape[0] != C:
        raise ValueError("scale must be (C,R) when no scale_row map is given")
    dev = Wts[0].device
    Qts = [torch.empty(C, R, dtype=torch.uint8, device=dev) for _ in range(k)]
    ring = lib.mq_gptq_loop_scratch_bytes(R)
    E = _ws.get(dev, ring * k, "loop")
    import ctypes as C_

    Ep = (C_.c_void_p * k)(*[E.data_ptr() + ring * i for i in range(k)])
    rc = lib.mq_gptq_loop_chol_grouped(k, _ptr_array(Wts), _ptr_array(W0ts), ldw, C, R, _ptr_array(Fs), ldf,
                                       _ptr_array(scales), lds, _ptr_array(scale_rows) if scale_rows is not None else None,
                                       None, qzero_const, maxq, _dt(round_dtype), block, _ptr_array(Qts), Ep, _stream(Wts[0]))
    check(rc, "mq_gptq_loop_chol_grouped")
    return Qts


def gptq_loop_(Wt: Tensor, U: Tensor, scale: Tensor, scale_row: Optional[Tensor], qzero: Optional[Tensor],
               qzero_const: float, maxq: float, round_dtype, block: int) -> Tensor:
    """Runs the loop in place on Wt (C,R); returns the codes Qt (C,R) uint8."""
    _dev(Wt, U, scale, scale_row, qzero)
    lib = _lib.load()
    C, R = Wt.shape
    for t in (Wt, U, scale) + ((qzero,) if qzero is not None else ()):
        if t.dtype != torch.float32 or t.stride(-1) != 1:
            raise ValueError("Wt, U, scale, qzero must be fp32 with unit inner stride")
    if qzero is not None and (qzero.shape != scale.shape or qzero.stride(0) != scale.stride(0)):
        raise ValueError("qzero must have the layout of scale")
    if scale_row is not None and (scale_row.dtype != torch.int32 or scale_row.numel() != C):
        raise ValueError("scale_row must be int32 of length C")
    if scale_row is None and scale.shape[0] != C:
        raise ValueError("scale must be (C,R) when no scale_row map is given")
    Qt = torch.empty(C, R, dtype=torch.uint8, device=Wt.device)
    E = _ws.get(Wt.device, lib.mq_gptq_loop_scratch_bytes(R), "loop")
    rc = lib.mq_gptq_loop(Wt.data_ptr(), Wt.stride(0), C, R, U.data_ptr(), U.stride(0), scale.data_ptr(),
                          scale.stride(0), _p(scale_row), _p(qzero), qzero_const, maxq, _dt(round_dtype), block,
                          Qt.data_ptr(), E.data_ptr(), _stream(Wt))
    check(rc, "mq_gptq_loop")
    return Qt


def gptq_loop_grouped_(Wts, Us, scales, scale_rows, qzero_const: float, maxq: float, round_dtype, block: int):
    """gptq_loop_ for several linears of one shape with one library call (lists of equal length; scale_rows: a list of
    int32 maps or None).  In place on every Wt; returns the list of code tensors Qt (C,R) uint8."""
    k = len(Wts)
    if not (len(Us) == len(scales) == k) or (scale_rows is not None and len(scale_rows) != k):
        raise ValueError("Wts, Us, scales, scale_rows must have the same length")
    if k == 0:
        return []
    _dev(*Wts, *Us, *scales, *(scale_rows or []))
    lib = _lib.load()
    C, R = Wts[0].shape
    ldw, ldu, lds = Wts[0].stride(0), Us[0].stride(0), scales[0].stride(0)
    for Wt, U, sc in zip(Wts, Us, scales):
        for t in (Wt, U, sc):
            if t.dtype != torch.float32 or t.stride(-1) != 1:
                raise ValueError("Wt, U, scale must be fp32 with unit inner stride")
        if Wt.shape != (C, R) or Wt.stride(0) != ldw or U.stride(0) != ldu or sc.stride(0) != lds:
            raise ValueError("all linears of a group share one shape and one set of pitches")
    if scale_rows is not None:
        for m in scale_rows:
            if m.dtype != torch.int32 or m.numel() != C:
                raise ValueError("scale_row must be int32 of length C")
    elif scales[0].shape[0] != C:
        raise ValueError("scale must be (C,R) when no scale_row map is given")
    dev = Wts[0].device
    Qts = [torch.empty(C, R, dtype=torch.uint8, device=dev) for _ in range(k)]
    ring = lib.mq_gptq_loop_scratch_bytes(R)
    E = _ws.get(dev, ring * k, "loop")
    import ctypes as C_

    Ep = (C_.c_void_p * k)(*[E.data_ptr() + ring * i for i in range(k)])
    rc = lib.mq_gptq_loop_grouped(k, _ptr_array(Wts), ldw, C, R, _ptr_array(Us), ldu, _ptr_array(scales), lds,
                                  _ptr_array(scale_rows) if scale_rows is not None else None, None, qzero_const, maxq,
                                  _dt(round_dtype), block, _ptr_array(Qts), Ep, _stream(Wts[0]))
    check(rc, "mq_gptq_loop_grouped")
    return Qts


def untranspose_codes(Qt: Tensor, perm_inv: Optional[Tensor] = None) -> Tensor:
    _dev(Qt, perm_inv)
    lib = _lib.load()
    C, R = Qt.shape
    codes = torch.empty(R, C, dtype=torch.uint8, device=Qt.device)
    rc = lib.mq_untranspose_codes(Qt.data_ptr(), R, C, _p(perm_inv), codes.data_ptr(), C, _stream(Qt))
    check(rc, "mq_untranspose_codes")
    return codes


# ---- (4) packing -------------------------------------------------------------------------------------
def pack_int4(codes: Tensor, zero: Optional[Tensor] = None, group_size: int = 0) -> Tensor:
    """codes (R,C) uint8 -> (R, ceil(C/8)) int32; zero (R,G) fp32 or None (= 8)."""
    _dev(codes, zero)
    lib = _lib.load()
    if codes.dtype != torch.uint8 or codes.dim() != 2:
        raise ValueError("codes must be (R,C) uint8")
    if codes.stride(1) != 1:
        codes = codes.contiguous()
    R, C = codes.shape
    words = (C + 7) // 8
    out = torch.empty(R, words, dtype=torch.int32, device=codes.device)
    if zero is not None:
        zero = zero.to(torch.float32).contiguous()
    rc = lib.mq_pack_int4(codes.data_ptr(), codes.stride(0), R, C, _p(zero), group_size, out.data_ptr(), words,
                          _stream(codes))
    check(rc, "mq_pack_int4")
    return out


def pack_from_qt(Qt: Tensor, perm_inv: Optional[Tensor] = None) -> Tensor:
    _dev(Qt, perm_inv)
    lib = _lib.load()
    C, R = Qt.shape
    words = (C + 7) // 8
    out = torch.empty(R, words, dtype=torch.int32, device=Qt.device)
    rc = lib.mq_pack_from_qt(Qt.data_ptr(), R, C, _p(perm_inv), out.data_ptr(), words, _stream(Qt))
    check(rc, "mq_pack_from_qt")
    return out


def dequant_fp8_block(W: Tensor, scale_inv: Tensor, dtype: torch.dtype) -> Tensor:
    """W (R,C) torch.float8_e4m3fn, scale_inv (ceil(R/128), ceil(C/128)) any float -> (R,C) bf16/fp16."""
    _dev(W, scale_inv)
    lib = _lib.load()
    if W.dtype != torch.float8_e4m3fn or W.dim() != 2:
        raise TypeError("W must be a 2-D torch.float8_e4m3fn tensor")
    if dtype not in (torch.bfloat16, torch.float16):
        raise TypeError("dtype must be bfloat16 or float16")
    R, C = W.shape
    if scale_inv.shape != ((R + 127) // 128, (C + 127) // 128):
        raise ValueError("scale_inv must have one entry per 128x128 block")
    if W.stride(1) != 1:
        W = W.contiguous()
    s = scale_inv.to(torch.float32).contiguous()
    out = torch.empty(R, C, dtype=dtype, device=W.device)
    rc = lib.mq_dequant_fp8_block(W.data_ptr(), W.stride(0), R, C, s.data_ptr(), s.stride(0), _dt(dtype), out.data_ptr(),
                                  out.stride(0), _stream(W))
    check(rc, "mq_dequant_fp8_block")
    return out


def swiglu(GU: Tensor) -> Tensor:
    """silu(GU[:, :I]) * GU[:, I:] for a (n, 2I) bf16/fp16 matrix of gate outputs followed by up outputs."""
    _dev(GU)
    lib = _lib.load()
    if GU.dim() != 2 or GU.dtype not in (torch.bfloat16, torch.float16) or GU.shape[1] % 16 or GU.stride(1) != 1:
        raise ValueError("GU must be (n, 2I) bf16/fp16 with unit column stride and I % 8 == 0")
    n, I = GU.shape[0], GU.shape[1] // 2
    out = torch.empty(n, I, dtype=GU.dtype, device=GU.device)
    check(lib.mq_swiglu(GU.data_ptr(), GU.stride(0), n, I, _dt(GU.dtype), out.data_ptr(), I, _stream(GU)), "mq_swiglu")
    return out


def swiglu_packed(G: Tensor, U: Tensor) -> PackedTokens:
    """silu(G) * U (both (n, I) bf16/fp16, rows may be strided: e.g. the two halves of one stacked GEMM output), same
    roundings as `swiglu`, written straight into the packed-token layout `hessian_syrk_packed_` reads."""
    _dev(G, U)
    lib = _lib.load()
    if (G.dim() != 2 or G.shape != U.shape or G.dtype != U.dtype or G.dtype not in (torch.bfloat16, torch.float16)
            or G.shape[1] % 8 or G.stride(1) != 1 or U.stride(1) != 1):
        raise ValueError("G and U must be (n, I) bf16/fp16 of one dtype with unit column stride and I % 8 == 0")
    n, I = G.shape
    nbytes = lib.mq_packed_tokens_bytes(n, I)
    out = torch.empty(max(nbytes, 16) // 2, dtype=G.dtype, device=G.device)
    check(lib.mq_swiglu_packed(G.data_ptr(), G.stride(0) if n > 1 else I, U.data_ptr(), U.stride(0) if n > 1 else I, n, I,
                               _dt(G.dtype), out.data_ptr(), _stream(G)), "mq_swiglu_packed")
    return PackedTokens(out, n, I, G.dtype)


def gemm_f32_(A, sam, sak, B, sbk, sbn, Cm, M, N, K, alpha=1.0, beta=0.0, tri=0, ktrim=0):
    _dev(A, B, Cm)
    lib = _lib.load()
    rc = lib.mq_gemm_f32(A.data_ptr(), sam, sak, B.data_ptr(), sbk, sbn, Cm.data_ptr(), Cm.stride(0), M, N, K, alpha,
                         beta, tri, ktrim, _stream(Cm))
    check(rc, "mq_gemm_f32")
    return Cm
