"""CPU restatement of MoE-Quant's GPTQ hot path (torch, fp32 unless stated).

THIS FILE IS TEST INFRASTRUCTURE.  It is the checker that the HIP kernels are
compared against and the "reference torch CPU path" that bench.py times as the
CPU baseline.  Nothing in the shipped package imports it; only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may.

Every function cites the reference lines (relative to the MoE-Quant tree) that
it follows.  The reference has no tests or golden vectors, so each function is
pinned by closed forms / invariants / brute force in tests/test_oracle_*.py:

  hessian_update ............ closed form (2/N) sum X^T X in fp64, batch-split invariance
  quantization_pre_step ..... special cases (no samples, NaN, dead channel)
  find_quantization_meta .... known answers (absmax 0.15 -> bf16(0.02), zero group -> bf16(1e-12))
  act_order_perm ............ argsort of distinct values is unique; perm_inv[perm] == arange
  hessian_inverse ........... torch's own LAPACK routines ARE the reference arithmetic; invariants
                              (upper, unit diagonal, (DU)^T(DU) H = I), diagonal H, 2x2 by hand
  gptq_loop ................. U = I -> plain round-to-nearest; fp64 un-blocked textbook GPTQ on tiny
                              shapes; block-size invariance; row independence; C % B != 0
  pack_int4 ................. closed form; known answer from upstream docstring ([1,2]@8bit -> 33409);
                              round trip.  compressed_tensors is absent from this image and un-pinned
                              by the reference (no version, no tests) -> "parity unpinned" beyond that.
  dequantize / relative_mse . closed form; tr(dH d^T) = (2/n)||X d^T||_F^2 against fp64 matmul
  mse_scale ................. brute force over the candidates in fp64 on tiny groups with well-separated
                              losses; the chosen candidate never loses to p = 1; all-zero group -> every loss
                              0 -> the LAST candidate wins (tie_break_left=False); a group that sits exactly
                              on the 4-bit grid keeps p = 1.  The bits of Triton's log/exp and the order of
                              its group sum decide near-ties between candidates: "parity unpinned" there.

  dequantize_weight_from_fp8  known answers for e4m3fn bytes (0x38 = 1, 0x7e = 448, 0x01 = 2^-9, 0x7f = NaN) through
                              torch's own fp8 cast; all 256 byte values against the format's definition; ragged
                              shapes against a per-element loop

Unpinnable by any means: torch.argsort tie order (unstable sort) and the exact
bits of Triton's fma / division on a GPU.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor

# ----------------------------------------------------------------------------------------------
# (a2) Hessian accumulation -- src/gptq.py:73-105
# ----------------------------------------------------------------------------------------------


def hessian_update(H: Optional[Tensor], num_samples: int, x: Tensor) -> Tuple[Tensor, int]:
    """H <- n0/(n0+n) H + 2/(n0+n) X^T X in fp32 (src/gptq.py:82-105)."""
    x = x.reshape(-1, x.shape[-1])  # src/gptq.py:86
    if H is None:
        H = torch.zeros((x.shape[-1], x.shape[-1]), dtype=torch.float32)  # src/gptq.py:82-83
    x = x.float()  # src/gptq.py:97
    n = x.shape[0]  # src/gptq.py:99
    beta = num_samples / (num_samples + n)  # src/gptq.py:101
    alpha = 2.0 / (num_samples + n)  # src/gptq.py:102
    H.addmm_(x.T, x, beta=beta, alpha=alpha)  # src/gptq.py:103
    return H, num_samples + n  # src/gptq.py:105


def hessian_fp64(batches) -> Tensor:
    """Ground truth (2/N) sum_b X_b^T X_b in float64 -- the 1e-5 Frobenius target."""
    acc, n = None, 0
    for x in batches:
        x = x.reshape(-1, x.shape[-1]).double()
        acc = x.T @ x if acc is None else acc + x.T @ x
        n += x.shape[0]
    return acc * (2.0 / n)


# ----------------------------------------------------------------------------------------------
# (a3) pre-step -- src/gptq.py:122-154
# ----------------------------------------------------------------------------------------------


def quantization_pre_step(H: Optional[Tensor], W: Tensor):
    """Returns (H, W32, issue_zero_samples, issue_nan_hessian) -- src/gptq.py:129-152 (untied, single process)."""
    d_col = W.shape[1]
    zero_samples = nan_hessian = False
    if H is None:  # src/gptq.py:129-134
        H = torch.eye(d_col, dtype=torch.float32)
        zero_samples = True
    if torch.isnan(H).any().item():  # src/gptq.py:141-143
        H = torch.eye(d_col, dtype=torch.float32)
        nan_hessian = True
    pruned = torch.diag(H) == 0  # src/gptq.py:145
    H[pruned, pruned] = 1  # src/gptq.py:146
    W = W.clone().float()  # src/gptq.py:149
    W[:, pruned] = 0  # src/gptq.py:152
    return H, W, zero_samples, nan_hessian


# ----------------------------------------------------------------------------------------------
# (a4) quantization grid -- src/quant_utils.py:52-101,195-240
# ----------------------------------------------------------------------------------------------


def round_fp(x: Tensor, dtype: Optional[torch.dtype]) -> Tensor:
    """src/quant_utils.py:52-53."""
    return x if dtype is None else x.to(dtype).to(x.dtype)


def find_quantization_meta(x: Tensor, bit_width: int, dtype: Optional[torch.dtype]):
    """Symmetric branch of src/quant_utils.py:75-96: reduction over the last dim."""
    maxq = torch.tensor(2**bit_width - 1, dtype=x.dtype)  # :87
    hi = x.amax(dim=-1)  # :89 (named x_min there; only |.| is used in the symmetric branch)
    lo = x.amin(dim=-1)  # :90
    scale = (2.0 / maxq) * torch.maximum(hi.abs(), lo.abs())  # :93
    scale = round_fp(scale + 1e-12, dtype)  # :94
    qzero = torch.full_like(scale, ((maxq + 1.0) * 0.5).item())  # :95
    return scale, qzero, maxq


def quantization_grid(W: Tensor, group_size: Optional[int], bits: int, dtype: Optional[torch.dtype],
                      mse: bool = False, max_shrink: float = 0.2, n_grid: int = 100, norm: float = 2.4):
    """Compact grid: scale (R,G) fp32 (bf16-exact), qzero (R,G), maxq () -- src/quant_utils.py:213-232.
    mse=True adds the scale search of :221-232 (what QuantizationScale.MSE selects)."""
    g = group_size or W.shape[-1]
    x = W.unflatten(-1, (-1, g))
    scale, qzero, maxq = find_quantization_meta(x, bits, dtype)
    if mse:
        scale = mse_scale(x.contiguous(), search_points(max_shrink, n_grid), scale, qzero, maxq, dtype, norm)
    return scale, qzero, maxq


def replicate_grid(scale: Tensor, qzero: Tensor, group_size: int):
    """(R,G) -> (R,C) as src/quant_utils.py:234-235."""
    return scale.repeat_interleave(group_size, dim=-1), qzero.repeat_interleave(group_size, dim=-1)


def mse_scale(x: Tensor, p: Tensor, scale: Tensor, qzero: Tensor, maxq: Tensor, dtype: Optional[torch.dtype] = None,
              norm: float = 2.4, chunk: int = 4096) -> Tensor:
    """Scale search of src/quant_utils.py:104-192: x (..., g) fp32, p (P,) shrink factors, scale/qzero (...).
    For every group the candidate scale round_fp(scale*p_i) minimising sum |dq(q(x)) - x|^norm wins, the last one
    among equals (tl.argmin(..., tie_break_left=False), :138); returns round_fp(scale * p[best]) (:140).
    |d|^norm is evaluated as exp(log|d| * norm) like tl_pow (:26-27); the quantizer is the Triton one
    (floor(v + 0.5), :30-49).  `scale` is not modified (the reference overwrites it in place)."""
    g = x.shape[-1]
    xs = x.reshape(-1, g)
    sc = scale.reshape(-1)
    qz = qzero.reshape(-1)
    out = torch.empty_like(sc)
    P = p.numel()
    for s0 in range(0, xs.shape[0], chunk):
        xb = xs[s0 : s0 + chunk][:, None, :]  # (B, 1, g)
        sp = round_fp(sc[s0 : s0 + chunk, None] * p[None, :], dtype)[:, :, None]  # (B, P, 1)  :135
        zb = qz[s0 : s0 + chunk, None, None]
        q = torch.floor(xb / sp + zb + 0.5).clamp(torch.zeros_like(maxq), maxq)  # tl_quantize
        dq = round_fp((q - zb) * sp, dtype)  # tl_dequantize
        loss = ((dq - xb).abs().log() * norm).exp().sum(dim=-1)  # (B, P)  :137
        best = (P - 1) - torch.argmin(loss.flip(-1), dim=-1)  # last index among equal minima
        out[s0 : s0 + chunk] = round_fp(sc[s0 : s0 + chunk] * p[best], dtype)  # :140
    return out.reshape(scale.shape)


def search_points(max_shrink: float = 0.2, n_grid: int = 100) -> Tensor:
    """src/quant_utils.py:222."""
    return torch.linspace(1, max_shrink, n_grid, dtype=torch.float32)


def quantize(x: Tensor, scale: Tensor, qzero: Tensor, maxq: Tensor, half_up: bool = True) -> Tensor:
    """half_up=True follows the Triton kernel used inside the loop (src/quant_utils.py:30-44:
    floor(x/s + z + 0.5)); half_up=False follows the torch helper (:57-58, round-half-even).
    The two differ only on exact ties."""
    v = x / scale + qzero
    r = torch.floor(v + 0.5) if half_up else v.round()
    return r.clamp(torch.zeros_like(maxq), maxq)


def dequantize(q: Tensor, scale: Tensor, qzero: Tensor, dtype: Optional[torch.dtype] = None) -> Tensor:
    """src/quant_utils.py:61-62 / :47-49."""
    return round_fp((q - qzero) * scale, dtype)


# ----------------------------------------------------------------------------------------------
# (a5) act-order -- src/gptq.py:179-187
# ----------------------------------------------------------------------------------------------


def act_order_perm(H: Tensor, act_order: bool):
    if act_order:
        perm = torch.argsort(H.diag(), descending=True)  # src/gptq.py:181
    else:
        perm = torch.arange(H.shape[0])  # src/gptq.py:183
    return perm, torch.argsort(perm)  # src/gptq.py:184


# ----------------------------------------------------------------------------------------------
# (a6) damped inverse factor -- src/gptq.py:220-243, src/linalg_utils.py:8-12
# ----------------------------------------------------------------------------------------------


def hessian_inverse(H: Tensor, W: Tensor, rel_damp: float, dtype=torch.float32):
    """H is modified in place (masking + damping) exactly as the reference does; returns
    (U, ok) with U = unit-diagonal upper factor; ok=False means the identity fallback fired.
    `dtype=torch.float64` gives the high-precision truth used to bound factorisation error."""
    d_col = H.shape[0]
    zero_cols = torch.nonzero(W.eq(0).all(dim=0))  # src/gptq.py:224
    H[zero_cols, :] = 0  # :228
    H[:, zero_cols] = 0  # :229
    H[zero_cols, zero_cols] = 1  # :230
    damp = rel_damp * torch.diag(H).mean()  # :233
    H[range(d_col), range(d_col)] += damp  # :234
    ok = True
    try:
        Hi = torch.cholesky_inverse(torch.linalg.cholesky(H.to(dtype)))  # src/linalg_utils.py:12
        U = torch.linalg.cholesky(Hi, upper=True)  # src/gptq.py:238
    except Exception:  # bare except at src/gptq.py:239
        U = torch.eye(d_col, dtype=dtype)
        ok = False
    U.div_(U.diag()[:, None])  # src/gptq.py:242
    return U, ok


# ----------------------------------------------------------------------------------------------
# (a7-a10) the blocked loop -- src/gptq_loop.py:141-148 with kernel bodies :28-40 and :77-88
# ----------------------------------------------------------------------------------------------


def _fma32(a: Tensor, b: Tensor, c: Tensor) -> Tensor:
    """fp32 fused multiply-add (tl.fma, src/gptq_loop.py:86): the fp32*fp32 product is exact in
    fp64; one fp64 add then one fp32 rounding (double rounding is possible only on ~2^-29 ties)."""
    return (a.double() * b.double() + c.double()).float()


def gptq_loop(
    weight: Tensor,
    hessian_inv: Tensor,
    scale: Tensor,
    qzero: Tensor,
    maxq: Tensor,
    dtype: Optional[torch.dtype],
    gptq_block_size: int = 128,
    half_up: bool = True,
    fused: bool = True,
    pre: Optional[Tensor] = None,
) -> Tensor:
    """weight (C,R) fp32 is modified in place to the dequantized values; returns codes (C,R) fp32.
    Mirrors gptq_loop_graph(direct=True), src/gptq_loop.py:141-148.
    pre (optional, (C,R) fp32): receives every column as it stands when its turn to be quantized comes (a
    by-product for tests that ask how close a rounding decision was; the arithmetic is untouched)."""
    C, R = weight.shape
    if gptq_block_size <= 0:  # src/gptq_loop.py:212-213
        gptq_block_size = C
    qweight = torch.empty_like(weight)
    err = torch.empty(gptq_block_size, R, dtype=weight.dtype)
    for i1 in range(0, C, gptq_block_size):
        i2 = min(i1 + gptq_block_size, C)
        for j in range(i1, i2):
            x = weight[j]
            if pre is not None:
                pre[j] = x
            q = quantize(x, scale[j], qzero[j], maxq, half_up)  # tl_quantize, src/gptq_loop.py:34
            y = dequantize(q, scale[j], qzero[j], dtype)  # tl_dequantize, :35
            e = y - x  # :36
            weight[j] = y  # :38
            qweight[j] = q  # :39
            err[j - i1] = e  # :40
            if j + 1 < i2:  # addvv: C[a,:] = fma(va[a], vb[:], C[a,:]), :77-88
                h = hessian_inv[j, j + 1 : i2, None]
                if fused:
                    weight[j + 1 : i2] = _fma32(h, e[None, :], weight[j + 1 : i2])
                else:
                    weight[j + 1 : i2] += h * e[None, :]
        if i2 < C:
            weight[i2:].addmm_(hessian_inv[i1:i2, i2:].t(), err[: i2 - i1], beta=1, alpha=1)  # :148
    return qweight


# ----------------------------------------------------------------------------------------------
# whole linear: GPTQ.quantize -- src/gptq.py:156-218
# ----------------------------------------------------------------------------------------------


def quantize_linear(
    W: Tensor,
    H: Optional[Tensor],
    bits: int = 4,
    group_size: Optional[int] = 128,
    rel_damp: float = 1e-2,
    block_size: Optional[int] = 128,
    act_order: bool = False,
    dtype: Optional[torch.dtype] = None,
    half_up: bool = True,
    inverse_dtype=torch.float32,
    mse: bool = False,
    keep_pre: bool = False,
    perm: Optional[Tensor] = None,
):
    """Returns dict(qweight u8 (R,C), scale (R,G), zero (R,G), U, perm, H (damped, permuted), ok).
    keep_pre: also `tie_distance` (R,C) fp32 in the original column order: how far x/s + zero + 0.5 was from the
    nearest integer when the column was quantized (0 = an exact tie of the rounding decision).
    perm: with act_order, the column order to use in place of this function's own argsort (src/gptq.py:181 sorts with
    an unstable sort: where diag(H) holds equal values their order is open, and a test that compares with a device run
    passes the order the device chose)."""
    dtype = dtype or W.dtype
    R, C = W.shape
    H, W32, zero_samples, nan_h = quantization_pre_step(H, W)
    g = group_size or C
    scale_g, zero_g, maxq = quantization_grid(W32, g, bits, dtype, mse=mse)  # src/gptq.py:171-178
    scale, zero = replicate_grid(scale_g, zero_g, g)
    if perm is not None and act_order:
        perm_inv = torch.argsort(perm)
    else:
        perm, perm_inv = act_order_perm(H, act_order)
    H = H[perm][:, perm]  # src/gptq.py:187
    U, ok = hessian_inverse(H, W32, rel_damp, inverse_dtype)  # :189
    U = U.float()
    Wt = W32.t()[perm].contiguous()  # :192
    st, zt = scale.t()[perm].contiguous(), zero.t()[perm].contiguous()
    pre = torch.empty_like(Wt) if keep_pre else None
    q = gptq_loop(Wt, U, st, zt, maxq, dtype, block_size or C, half_up, pre=pre)
    qweight = q[perm_inv].t().contiguous().to(torch.uint8)  # :199
    extra = {}
    if keep_pre:
        v = pre / st + zt + 0.5
        extra["tie_distance"] = (v - torch.round(v)).abs()[perm_inv].t().contiguous()
        extra["order_position"] = perm_inv  # position of original column c in the loop's walking order
    return dict(
        **extra,
        qweight=qweight,
        scale=scale[:, ::g].to(dtype),  # :201
        zero=zero[:, ::g].to(dtype),  # :202
        U=U,
        perm=perm,
        H=H,
        ok=ok,
        issue_zero_samples=zero_samples,
        issue_nan_hessian=nan_h,
    )


# ----------------------------------------------------------------------------------------------
# (a12-a13) dequantize + error metric -- src/quant_utils.py:243-264
# ----------------------------------------------------------------------------------------------


def dequantize_linear_weight(qweight: Tensor, scale: Tensor, zero: Tensor, perm: Optional[Tensor] = None) -> Tensor:
    R = qweight.shape[0]
    s = scale.view(R, -1, 1)
    z = zero.view(R, -1, 1)
    w = dequantize(qweight.view(R, s.shape[1], -1), s, z).view_as(qweight)  # :250 (u8 - bf16 -> bf16)
    if perm is not None:
        w = w[:, perm.argsort()]  # :253-255
    return w


def relative_mse(q: Tensor, w: Tensor, H: Optional[Tensor] = None) -> Tensor:
    d = q - w
    if H is None:
        return d.pow(2).mean() / w.pow(2).mean()  # :262
    return d.mm(H).mul(d).mean() / (w.mm(H).mul(w).mean() + 1e-6)  # :264


# ----------------------------------------------------------------------------------------------
# (a14) packing -- pack_quantized_model.py:57-75 + compressed_tensors.pack_to_int32 (absent here)
# ----------------------------------------------------------------------------------------------


def pack_to_int32(value: Tensor, num_bits: int) -> Tensor:
    """Published algorithm of compressed_tensors.compressors.pack_to_int32 (no version pinned by the
    reference, package absent from this image): int8 input, offset by 2^(bits-1) to unsigned,
    pad the last dim to a multiple of 32/bits, element i of each word in bits [bits*i, bits*i+bits)."""
    if value.dtype != torch.int8:
        raise ValueError("Tensor must be quantized to torch.int8 before packing")
    if num_bits > 8:
        raise ValueError("Packing is only supported for less than 8 bits")
    u = (value.to(torch.int16) + (1 << (num_bits - 1))).to(torch.int64) & ((1 << num_bits) - 1)
    pf = 32 // num_bits
    rows, cols = u.shape
    pad = (-cols) % pf
    if pad:
        u = torch.nn.functional.pad(u, (0, pad))
    u = u.view(rows, -1, pf)
    shifts = torch.arange(pf, dtype=torch.int64) * num_bits
    word = (u << shifts).sum(-1)  # disjoint bit fields: sum == or
    word = torch.where(word >= 2**31, word - 2**32, word)
    return word.to(torch.int32)


def unpack_from_int32(packed: Tensor, num_bits: int, shape) -> Tensor:
    pf = 32 // num_bits
    w = packed.to(torch.int64) & 0xFFFFFFFF
    shifts = torch.arange(pf, dtype=torch.int64) * num_bits
    u = (w[..., None] >> shifts) & ((1 << num_bits) - 1)
    u = u.reshape(packed.shape[0], -1)[:, : shape[1]]
    return (u - (1 << (num_bits - 1))).to(torch.int8)


def pack_weight(weight: dict, bits: int, sym: bool, group_size: Optional[int] = None) -> dict:
    """pack_quantized_model.py:57-75."""
    qweight, scale, zero = weight["qweight"], weight["scale"], weight["zero"]
    group_size = group_size or qweight.shape[-1]
    shifted = qweight.to(torch.int8) - zero.repeat_interleave(group_size, dim=-1).to(torch.int8)  # :66
    out = {
        "weight_packed": pack_to_int32(shifted, bits),  # :67
        "weight_shape": torch.tensor(qweight.shape),  # :70
        "weight_scale": scale,  # :71
    }
    if not sym:
        out["weight_zero_point"] = weight["zero"]  # :73-74
    return out


# ----------------------------------------------------------------------------------------------
# checkpoint ingest -- src/quant_utils.py:267-298
# ----------------------------------------------------------------------------------------------


def dequantize_weight_from_fp8(W: Tensor, s: Tensor, g: int = 128) -> Tensor:
    """src/quant_utils.py:267-284, statement by statement (pad, view as blocks, multiply, crop)."""
    import math

    import torch.nn.functional as F

    d_out, d_in = W.shape
    pad_out = math.ceil(d_out / g) * g - d_out
    pad_in = math.ceil(d_in / g) * g - d_in
    W = F.pad(W, (0, pad_in, 0, pad_out))
    d_out_pad, d_in_pad = W.shape
    W = W.view(d_out_pad // g, g, d_in_pad // g, g)
    s = s.view(d_out_pad // g, 1, d_in_pad // g, 1)
    W = (W * s).view(d_out_pad, d_in_pad)
    return W[:d_out, :d_in]


def dequantize_fp8_entry(W8: Tensor, scale_inv: Tensor, dtype: torch.dtype) -> Tensor:
    """What dequantize_state_dict does to one (weight, weight_scale_inv) pair, src/quant_utils.py:292-296."""
    return dequantize_weight_from_fp8(W8.to(dtype), scale_inv.to(dtype))
