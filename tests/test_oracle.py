"""Pins for the CPU oracle.  The reference has no tests or golden vectors, so every function of
oracle/gptq_oracle.py is checked against something it does not itself compute: closed forms, known
answers, fp64 brute force, invariants, and the independently written C restatement."""
import ctypes
import math
import os

import numpy as np
import pytest
import torch

from moe_quant_amd import synth
from oracle import gptq_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _rand(shape, seed, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


# ------------------------------------------------------------------ a2 Hessian
def test_hessian_closed_form_and_batch_split():
    X = synth.activations_outlier(700, 96, 1)
    H1, n1 = O.hessian_update(None, 0, X)
    H64 = (2.0 / 700) * (X.double().T @ X.double())
    assert n1 == 700
    assert ((H1.double() - H64).norm() / H64.norm()).item() < 1e-6
    assert torch.allclose(H1, H1.T, rtol=0, atol=1e-4 * H1.abs().max().item())
    H, n = None, 0
    for chunk in (X[:100], X[100:101], X[101:450], X[450:]):
        H, n = O.hessian_update(H, n, chunk)
    assert n == 700
    assert ((H - H1).norm() / H1.norm()).item() < 1e-6
    assert ((O.hessian_fp64([X[:300], X[300:]]) - H64).norm() / H64.norm()).item() < 1e-14
    # brute force on a tiny case, 3-D input is flattened over leading dims
    x = torch.tensor([[[1.0, 2.0], [3.0, 4.0]], [[0.5, -1.0], [0.0, 2.0]]]).bfloat16()
    Hb, nb = O.hessian_update(None, 0, x)
    want = torch.zeros(2, 2)
    for t in x.reshape(-1, 2).float():
        want += torch.outer(t, t)
    assert nb == 4 and torch.allclose(Hb, want * 0.5)


# ------------------------------------------------------------------ a3 pre-step
def test_pre_step_special_cases():
    W = _rand((4, 6), 2).bfloat16()
    H, W32, zs, nan = O.quantization_pre_step(None, W)
    assert zs and not nan and torch.equal(H, torch.eye(6)) and W32.dtype == torch.float32
    Hn = torch.eye(6)
    Hn[2, 3] = float("nan")
    H, _, zs, nan = O.quantization_pre_step(Hn, W)
    assert nan and not zs and torch.equal(H, torch.eye(6))
    X = _rand((50, 6), 3).bfloat16()
    X[:, 4] = 0
    Hd, _ = O.hessian_update(None, 0, X)
    H, W32, zs, nan = O.quantization_pre_step(Hd, W)
    assert not zs and not nan and H[4, 4] == 1 and torch.all(W32[:, 4] == 0)
    assert torch.equal(W32[:, :4], W.float()[:, :4])


# ------------------------------------------------------------------ a4 grid
def test_grid_known_answers():
    w = torch.zeros(2, 256)
    w[0, 5] = 0.15  # |max| 0.15 -> (2/15)*0.15 = 0.02 -> bf16 0.02001953125
    w[0, 130] = -0.3  # second group uses |min|
    s, z, maxq = O.quantization_grid(w, 128, 4, torch.bfloat16)
    assert maxq.item() == 15.0 and torch.all(z == 8.0) and s.shape == (2, 2)
    assert s[0, 0].item() == 0.02001953125
    assert s[0, 1].item() == torch.tensor(np.float32(2.0) / np.float32(15.0) * np.float32(0.3)).bfloat16().float().item()
    zero_scale = torch.tensor(1e-12).bfloat16().float().item()
    assert s[1, 0].item() == zero_scale and abs(zero_scale - 1.00186e-12) < 1e-16
    assert torch.equal(s, s.bfloat16().float())  # bf16-exact
    sr, zr = O.replicate_grid(s, z, 128)
    assert sr.shape == (2, 256) and torch.all(sr[0, :128] == s[0, 0]) and torch.all(sr[0, 128:] == s[0, 1])
    # dtype=None keeps fp32; per-row grid when group_size is None
    s32, _, _ = O.quantization_grid(w, None, 4, None)
    assert s32.shape == (2, 1) and s32[0, 0].item() == np.float32(np.float32(2.0) / np.float32(15.0) * np.float32(0.3) + np.float32(1e-12))


def test_quantize_rounding_modes_differ_only_on_ties():
    maxq = torch.tensor(15.0)
    s, z = torch.tensor(1.0), torch.tensor(8.0)
    x = torch.tensor([0.5, 1.5, -0.5, 0.49, 9.0, -20.0])
    up = O.quantize(x, s, z, maxq, half_up=True)
    ev = O.quantize(x, s, z, maxq, half_up=False)
    assert up.tolist() == [9.0, 10.0, 8.0, 8.0, 15.0, 0.0]
    assert ev.tolist() == [8.0, 10.0, 8.0, 8.0, 15.0, 0.0]
    y = O.dequantize(torch.tensor(11.0), torch.tensor(0.0200195), z, torch.bfloat16)
    assert y.item() == torch.tensor(3 * 0.0200195).bfloat16().float().item()


# ------------------------------------------------------------------ a5 perm
def test_act_order_perm():
    H = torch.diag(torch.tensor([3.0, 9.0, 1.0, 5.0]))
    perm, inv = O.act_order_perm(H, True)
    assert perm.tolist() == [1, 3, 0, 2] and torch.equal(inv[perm], torch.arange(4))
    perm, inv = O.act_order_perm(H, False)
    assert perm.tolist() == [0, 1, 2, 3]


# ------------------------------------------------------------------ a6 inverse factor
def test_hessian_inverse_invariants_and_special_cases():
    X = synth.activations_outlier(400, 64, 4)
    H, _ = O.hessian_update(None, 0, X)
    W = _rand((8, 64), 5, 0.02)
    Hd = H.clone()
    U, ok = O.hessian_inverse(Hd, W, 0.01)
    assert ok and torch.equal(U, torch.triu(U)) and torch.allclose(U.diag(), torch.ones(64))
    assert torch.allclose(Hd.diag(), H.diag() + 0.01 * H.diag().mean())  # damping applied in place
    M = U.double() @ Hd.double() @ U.double().T  # = D^-2 (diagonal, positive)
    off = M - torch.diag(M.diag())
    assert off.abs().max().item() < 1e-4 * M.diag().abs().max().item() and torch.all(M.diag() > 0)
    # fp64 path agrees with fp32 path to fp32 accuracy
    U64, _ = O.hessian_inverse(H.clone(), W, 0.01, torch.float64)
    assert ((U.double() - U64).norm() / U64.norm()).item() < 1e-5
    # diagonal H -> identity
    Ud, ok = O.hessian_inverse(torch.diag(torch.tensor([4.0, 1.0, 9.0])), torch.ones(2, 3), 0.0)
    assert ok and torch.allclose(Ud, torch.eye(3))
    # 2x2 by hand: H=[[a,b],[b,c]] -> U01 = -b/c  (regression coefficient of x0 on x1, sign flipped)
    a, b, c = 4.0, 1.0, 2.0
    U2, ok = O.hessian_inverse(torch.tensor([[a, b], [b, c]]), torch.ones(1, 2), 0.0)
    assert ok and abs(U2[0, 1].item() - (-b / c)) < 1e-6 and U2[1, 0].item() == 0
    # not positive definite -> identity fallback
    Un, ok = O.hessian_inverse(torch.tensor([[1.0, 2.0], [2.0, 1.0]]), torch.ones(1, 2), 0.0)
    assert (not ok) and torch.equal(Un, torch.eye(2))
    # an all-zero weight column masks that row/column of H
    Wz = W.clone()
    Wz[:, 7] = 0
    Hz = H.clone()
    Uz, ok = O.hessian_inverse(Hz, Wz, 0.01)
    assert ok and torch.all(Uz[7, 8:] == 0) and torch.all(Uz[:7, 7] == 0)


# ------------------------------------------------------------------ a7-a10 loop
def _loop_inputs(R, C, seed, g):
    W = synth.weight(R, C, seed).float()
    X = synth.activations_outlier(2 * C, C, seed + 1)
    H, _ = O.hessian_update(None, 0, X)
    s, z, maxq = O.quantization_grid(W, g, 4, torch.bfloat16)
    sr, zr = O.replicate_grid(s, z, g)
    U, _ = O.hessian_inverse(H.clone(), W, 0.01)
    return W, H, U.contiguous(), s, sr, zr, maxq


def test_loop_identity_is_round_to_nearest():
    W, H, U, s, sr, zr, maxq = _loop_inputs(16, 64, 10, 32)
    Wt = W.t().contiguous()
    q = O.gptq_loop(Wt, torch.eye(64), sr.t().contiguous(), zr.t().contiguous(), maxq, torch.bfloat16, 16)
    want = torch.floor(W.t() / sr.t() + 8.5).clamp(0, 15)
    assert torch.equal(q, want)
    assert torch.equal(Wt, ((q - 8) * sr.t()).bfloat16().float())


def _textbook_gptq_fp64(W, H, scale_rep, rel_damp):
    """Frantar et al., Algorithm 1, un-blocked, fp64, error (w - q)/d with the un-normalised upper
    Cholesky factor of H^-1 -- a different formulation from the one the oracle restates."""
    W = W.double().clone()
    H = H.double().clone()
    C = H.shape[0]
    H.diagonal().add_(rel_damp * H.diag().mean())
    Hinv = torch.linalg.cholesky(torch.linalg.inv(H), upper=True)
    Q = torch.zeros_like(W)
    s = scale_rep.double()
    for j in range(C):
        w = W[:, j]
        q = torch.clamp(torch.floor(w / s[:, j] + 8.5), 0, 15)
        Q[:, j] = q
        y = ((q - 8) * s[:, j]).float().bfloat16().double()  # dequantized value as stored: bf16
        err = (w - y) / Hinv[j, j]
        W[:, j + 1:] -= err[:, None] * Hinv[j, j + 1:][None, :]
    return Q


def test_loop_matches_fp64_textbook_gptq():
    total = same = 0
    for seed in (20, 21, 22):
        W, H, U, s, sr, zr, maxq = _loop_inputs(24, 48, seed, 16)
        q = O.gptq_loop(W.t().contiguous(), U, sr.t().contiguous(), zr.t().contiguous(), maxq, torch.bfloat16, 16)
        ref = _textbook_gptq_fp64(W, H, sr, 0.01)
        total += q.numel()
        same += (q.t() == ref).sum().item()
    # fp32 vs fp64 may flip a code that sits within 1e-6 of a rounding boundary; anything structural
    # (sign, index, missing term) would scramble most codes
    assert same / total > 0.995, same / total


def test_loop_block_size_invariance_and_row_independence():
    W, H, U, s, sr, zr, maxq = _loop_inputs(32, 160, 30, 32)
    st, zt = sr.t().contiguous(), zr.t().contiguous()
    base = O.gptq_loop(W.t().contiguous(), U, st, zt, maxq, torch.bfloat16, 128)
    assert base.min() >= 0 and base.max() <= 15
    for B in (1, 16, 48, 160, -1):  # 48 and 128 do not divide 160: ragged last block
        q = O.gptq_loop(W.t().contiguous(), U, st, zt, maxq, torch.bfloat16, B)
        assert (q == base).float().mean().item() > 0.995
    rows = torch.tensor([3, 17, 30])
    sub = O.gptq_loop(W[rows].t().contiguous(), U, st[:, rows].contiguous(), zt[:, rows].contiguous(), maxq,
                      torch.bfloat16, 128)
    assert torch.equal(sub, base[:, rows])
    # non-fused multiply-add differs from the fused one by rounding only
    q2 = O.gptq_loop(W.t().contiguous(), U, st, zt, maxq, torch.bfloat16, 128, fused=False)
    assert (q2 == base).float().mean().item() > 0.995


def _c_oracle():
    path = os.path.join(ROOT, "oracle", "libgptq_ref.so")
    if not os.path.exists(path):
        pytest.skip("oracle/libgptq_ref.so not built (run `make -C oracle`)")
    lib = ctypes.CDLL(path)
    lib.mq_ref_gptq_loop.restype = ctypes.c_int
    lib.mq_ref_gptq_loop.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                     ctypes.c_void_p, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.mq_ref_pack_int4.restype = None
    lib.mq_ref_pack_int4.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    return lib


def test_c_restatement_agrees_with_torch_oracle():
    lib = _c_oracle()
    W, H, U, s, sr, zr, maxq = _loop_inputs(48, 192, 40, 64)
    st, zt = sr.t().contiguous(), zr.t().contiguous()
    for B in (192, 64):
        Wt_t = W.t().contiguous()
        q_t = O.gptq_loop(Wt_t, U, st, zt, maxq, torch.bfloat16, B)
        Wt_c = W.t().contiguous()
        q_c = torch.empty_like(Wt_c)
        rc = lib.mq_ref_gptq_loop(Wt_c.data_ptr(), 192, 48, U.data_ptr(), st.data_ptr(), zt.data_ptr(), 15.0, 1, B,
                                  q_c.data_ptr())
        assert rc == 0
        if B == 192:  # no trailing GEMM: every operation is elementwise with one rounding -> bit identical
            assert torch.equal(q_c, q_t) and torch.equal(Wt_c, Wt_t)
        else:  # the BLAS call of the torch path sums in its own order
            assert (q_c == q_t).float().mean().item() > 0.995
    codes = torch.randint(0, 16, (9, 44), dtype=torch.uint8, generator=torch.Generator().manual_seed(1))
    out = torch.empty(9, 6, dtype=torch.int32)
    lib.mq_ref_pack_int4(codes.data_ptr(), 9, 44, out.data_ptr())
    assert torch.equal(out, O.pack_to_int32(codes.to(torch.int8) - 8, 4))


# ------------------------------------------------------------------ a11-a13
def test_dequantize_linear_weight_and_relative_mse():
    q = torch.randint(0, 16, (6, 64), dtype=torch.uint8, generator=torch.Generator().manual_seed(2))
    s = (_rand((6, 2), 3).abs() * 0.01 + 0.001).bfloat16()
    z = torch.full((6, 2), 8.0).bfloat16()
    w = O.dequantize_linear_weight(q, s, z)
    want = ((q.float() - 8.0) * s.float().repeat_interleave(32, 1)).bfloat16()
    assert w.dtype == torch.bfloat16 and torch.equal(w, want)
    perm = torch.randperm(64, generator=torch.Generator().manual_seed(4))
    assert torch.equal(O.dequantize_linear_weight(q, s, z, perm), want[:, perm.argsort()])
    X = _rand((300, 64), 5).double()
    H = (2.0 / 300) * X.T @ X
    W = _rand((6, 64), 6, 0.02).double()
    D = w.double() - W
    lhs = O.relative_mse(w.double(), W, H).item()
    num = (X @ D.T).pow(2).sum() * (2.0 / 300) / D.numel()
    den = (X @ W.T).pow(2).sum() * (2.0 / 300) / W.numel() + 1e-6
    assert abs(lhs - (num / den).item()) < 1e-9 * abs(lhs)
    assert abs(O.relative_mse(w.double(), W).item() - (D.pow(2).mean() / W.pow(2).mean()).item()) < 1e-12


# ------------------------------------------------------------------ a14 packing
def test_pack_known_answers_and_round_trip():
    # upstream docstring example: [1, 2] at 8 bits -> 129 + 130*256 = 33409 (low element in low bits)
    assert O.pack_to_int32(torch.tensor([[1, 2]], dtype=torch.int8), 8).tolist() == [[33409]]
    # 4 bits by hand: values -8..-1 -> nibbles 0..7 -> 0x76543210
    v = torch.arange(-8, 0, dtype=torch.int8)[None]
    assert O.pack_to_int32(v, 4).tolist() == [[0x76543210]]
    # top nibble >= 8 wraps into the sign bit of int32
    v = torch.tensor([[0, 0, 0, 0, 0, 0, 0, 7]], dtype=torch.int8)
    assert O.pack_to_int32(v, 4).tolist() == [[(0xF8888888) - (1 << 32)]]
    q = torch.randint(-8, 8, (5, 19), dtype=torch.int8, generator=torch.Generator().manual_seed(7))
    p = O.pack_to_int32(q, 4)
    assert p.shape == (5, 3) and p.dtype == torch.int32
    assert torch.equal(O.unpack_from_int32(p, 4, q.shape), q)
    with pytest.raises(ValueError):
        O.pack_to_int32(q.to(torch.int32), 4)
    out = O.pack_weight({"qweight": (q + 8).to(torch.uint8), "scale": torch.ones(5, 1), "zero": torch.full((5, 1), 8.0)},
                        4, True, None)
    assert torch.equal(out["weight_packed"], p) and out["weight_shape"].tolist() == [5, 19]
    assert "weight_zero_point" not in out


# ------------------------------------------------------------------ whole linear
def test_quantize_linear_end_to_end_properties():
    case = synth.config1(scale=1 / 16)  # 128 x 512 weights (R floor is 128), 512 tokens
    H, n = O.hessian_update(None, 0, case.X)
    out = O.quantize_linear(case.W, H.clone())
    q, s, z = out["qweight"], out["scale"], out["zero"]
    R, C = case.W.shape
    assert q.shape == (R, C) and q.dtype == torch.uint8 and s.shape == (R, C // 128) and s.dtype == torch.bfloat16
    assert torch.all(z == 8) and out["ok"]
    dq = O.dequantize_linear_weight(q, s, z).double()
    rtn = O.quantize_linear(case.W, None)  # identity Hessian = round to nearest
    assert rtn["issue_zero_samples"]
    dq_rtn = O.dequantize_linear_weight(rtn["qweight"], rtn["scale"], rtn["zero"]).double()
    H64 = O.hessian_fp64([case.X])
    e_gptq = O.relative_mse(dq, case.W.double(), H64).item()
    e_rtn = O.relative_mse(dq_rtn, case.W.double(), H64).item()
    assert e_gptq < e_rtn  # the whole point of GPTQ
    # act-order: codes come back in original column order
    out2 = O.quantize_linear(case.W, H.clone(), act_order=True)
    dq2 = O.dequantize_linear_weight(out2["qweight"], out2["scale"], out2["zero"]).double()
    assert O.relative_mse(dq2, case.W.double(), H64).item() < e_rtn
    assert torch.equal(out2["scale"], s)  # static scales do not depend on the order


# ---------------------------------------------------------------- MSE scale search (src/quant_utils.py:104-192)
def _brute_mse_scale(x, p, scale, qzero, maxq, norm):
    """Independent restatement in Python floats (fp64) with an explicit loop and an explicit last-minimum rule."""
    import math

    def bf16(v):
        return torch.tensor(v, dtype=torch.float32).to(torch.bfloat16).float().item()

    out = []
    for xi, s0, z in zip(x.tolist(), scale.tolist(), qzero.tolist()):
        best, best_loss = None, None
        for pi in p.tolist():
            sp = bf16(torch.tensor(s0, dtype=torch.float32).mul(torch.tensor(pi, dtype=torch.float32)).item())
            loss = 0.0
            for v in xi:
                q = min(max(math.floor(v / sp + z + 0.5), 0.0), maxq)
                d = abs(bf16((q - z) * sp) - v)
                loss += d**norm if d > 0 else 0.0
            if best_loss is None or loss <= best_loss:
                best, best_loss = sp, loss
        out.append(best)
    return torch.tensor(out)


def test_mse_scale_matches_brute_force_on_tiny_groups():
    g = torch.Generator().manual_seed(7)
    x = torch.randn(12, 16, generator=g) * 0.03
    x[:, 0] *= 4.0  # an outlier per group: shrinking the scale pays off
    p = O.search_points(0.2, 25)
    scale, qzero, maxq = O.find_quantization_meta(x, 4, torch.bfloat16)
    got = O.mse_scale(x, p, scale, qzero, maxq, torch.bfloat16, 2.4)
    want = _brute_mse_scale(x, p, scale, qzero, maxq.item(), 2.4)
    assert torch.equal(got, want)
    assert (got < scale).any()  # the search did move some scales


def test_mse_scale_special_cases():
    p = O.search_points()
    maxq = torch.tensor(15.0)
    # all-zero group: every candidate has loss 0, the last one wins (tie_break_left=False)
    x = torch.zeros(1, 128)
    scale, qzero, _ = O.find_quantization_meta(x, 4, torch.bfloat16)
    got = O.mse_scale(x, p, scale, qzero, maxq, torch.bfloat16)
    assert torch.equal(got, (scale * p[-1]).to(torch.bfloat16).float())
    # a group that already sits on the grid of its absmax scale: p = 1 has loss 0 and is the only such candidate
    s0 = torch.tensor([0.015625])
    x = ((torch.arange(128) % 16).float() - 8.0) * s0
    x = x[None]  # values (k - 8) * s0, k = 0..15: exactly the 4-bit grid of scale s0
    x[0, 1] = 7.0 * s0
    scale = torch.tensor([0.015625])
    got = O.mse_scale(x, p, scale, torch.tensor([8.0]), maxq, torch.bfloat16)
    assert torch.equal(got, scale)
    # the winner never loses to the absmax scale itself
    g = torch.Generator().manual_seed(3)
    x = torch.randn(64, 128, generator=g) * 0.02
    scale, qzero, _ = O.find_quantization_meta(x, 4, torch.bfloat16)
    got = O.mse_scale(x, p, scale, qzero, maxq, torch.bfloat16)

    def loss(sc):
        q = torch.floor(x / sc[:, None] + 8.5).clamp(0, 15)
        dq = ((q - 8.0) * sc[:, None]).to(torch.bfloat16).float()
        return (dq - x).abs().double().pow(2.4).sum(-1)

    assert torch.all(loss(got) <= loss(scale) * (1 + 1e-6))


# ---------------------------------------------------------------- FP8 block dequantisation (src/quant_utils.py:267-298)
def test_fp8_dequant_oracle_pins():
    b = torch.arange(256, dtype=torch.uint8)
    vals = b.view(torch.float8_e4m3fn).float()
    # the format's definition: sign, 4-bit exponent (bias 7), 3-bit mantissa, no infinities, S.1111.111 = NaN
    want = []
    for x in range(256):
        sgn, e, m = (-1.0 if x & 0x80 else 1.0), (x >> 3) & 15, x & 7
        if e == 15 and m == 7:
            want.append(float("nan"))
        elif e == 0:
            want.append(sgn * m * 2.0**-9)
        else:
            want.append(sgn * (1 + m / 8) * 2.0 ** (e - 7))
    want = torch.tensor(want)
    assert torch.equal(torch.nan_to_num(vals, nan=-77.0), torch.nan_to_num(want, nan=-77.0))
    assert vals[0x38] == 1.0 and vals[0x7E] == 448.0 and vals[0x01] == 2.0**-9 and torch.isnan(vals[0x7F])
    # ragged shape against a per-element loop
    g = torch.Generator().manual_seed(5)
    W8 = torch.randint(0, 256, (130, 260), generator=g, dtype=torch.uint8)
    W8[W8 == 0x7F] = 0
    W8[W8 == 0xFF] = 0
    W8 = W8.view(torch.float8_e4m3fn)
    s = torch.rand(2, 3, generator=g) * 0.01 + 1e-4
    got = O.dequantize_fp8_entry(W8, s, torch.bfloat16)
    assert got.dtype == torch.bfloat16 and got.shape == (130, 260)
    sb = s.to(torch.bfloat16)
    for r, c in [(0, 0), (127, 127), (128, 128), (129, 259), (5, 200), (129, 0)]:
        w = W8[r, c].to(torch.bfloat16)
        assert got[r, c] == w * sb[r // 128, c // 128]
