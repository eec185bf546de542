"""Kernel-level parity: each C-ABI entry point against the CPU oracle on the same seeded inputs."""
import pytest
import torch

from moe_quant_amd import ops, synth
from oracle import gptq_oracle as O

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)


def _rand(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


# ---------------------------------------------------------------- fp32 MFMA GEMM building block
@pytest.mark.parametrize("a_kc,b_kc", [(True, True), (True, False), (False, True), (False, False)])
@pytest.mark.parametrize("M,N,K", [(128, 128, 128), (300, 200, 72), (64, 576, 128), (513, 129, 17)])
def test_gemm_f32_layouts(dev, a_kc, b_kc, M, N, K):
    _say(f"gemm a_kc={a_kc} b_kc={b_kc} {M}x{N}x{K}")
    A = _rand((M, K), 1)
    B = _rand((K, N), 2)
    C0 = _rand((M, N), 3)
    Ad = (A if a_kc else A.t().contiguous()).to(dev)
    Bd = (B.t().contiguous() if b_kc else B).to(dev)
    Cd = C0.clone().to(dev)
    sam, sak = (K, 1) if a_kc else (1, M)
    sbk, sbn = (1, K) if b_kc else (N, 1)
    ops.gemm_f32_(Ad, sam, sak, Bd, sbk, sbn, Cd, M, N, K, alpha=-0.5, beta=2.0)
    ref = 2.0 * C0.double() - 0.5 * (A.double() @ B.double())
    err = (Cd.cpu().double() - ref).abs().max().item()
    assert err < 1e-4 * max(1.0, ref.abs().max().item()), err


@pytest.mark.parametrize("a_kc,b_kc", [(True, True), (True, False), (False, True), (False, False)])
@pytest.mark.parametrize("K", [16, 32, 48, 80, 256])
def test_gemm_f32_interior_tiles_short_and_odd_k(dev, a_kc, b_kc, K):
    """Interior 128x128 tiles (the bf16-piece core with two k-steps in flight) with 1, 2, 3, 5 and 16 k-steps:
    the pipeline's start and tail.  Against fp64 the error stays at fp32 rounding level."""
    M, N = 256, 384
    _say(f"gemm interior a_kc={a_kc} b_kc={b_kc} K={K}")
    A = _rand((M, K), 11) * (1.0 + 100.0 * torch.rand(M, 1, generator=torch.Generator().manual_seed(12)))
    B = _rand((K, N), 13)
    C0 = _rand((M, N), 14)
    Ad = (A if a_kc else A.t().contiguous()).to(dev)
    Bd = (B.t().contiguous() if b_kc else B).to(dev)
    Cd = C0.clone().to(dev)
    sam, sak = (K, 1) if a_kc else (1, M)
    sbk, sbn = (1, K) if b_kc else (N, 1)
    ops.gemm_f32_(Ad, sam, sak, Bd, sbk, sbn, Cd, M, N, K, alpha=-1.0, beta=1.0)
    ref = C0.double() - A.double() @ B.double()
    mag = C0.double().abs() + A.double().abs() @ B.double().abs()
    rel = ((Cd.cpu().double() - ref).abs() / mag).max().item()
    assert rel < 4e-7, rel


def test_gemm_f32_interior_tiles_wide_dynamic_range(dev):
    """Magnitudes from 1e-12 to 1e12 inside one row: every piece product is exact, but a matrix instruction
    aligns its 16 addends to the largest before adding, so the error is a few ulp of the largest terms rather
    than of each term.  It stays within 2e-6 of sum |a||b| (K = 512; the worst-case bound of any fp32 summation
    is K * 6e-8 = 3e-5) and is compared with torch's fp32 product of the same operands."""
    M, N, K = 256, 256, 512
    g = torch.Generator().manual_seed(21)
    A = torch.randn(M, K, generator=g) * torch.pow(10.0, torch.rand(M, K, generator=g) * 24 - 12)
    B = torch.randn(K, N, generator=g) * torch.pow(10.0, torch.rand(K, N, generator=g) * 24 - 12)
    Cd = torch.zeros(M, N, device=dev)
    ops.gemm_f32_(A.to(dev), K, 1, B.t().contiguous().to(dev), 1, K, Cd, M, N, K, alpha=1.0, beta=0.0)
    ref = A.double() @ B.double()
    mag = A.double().abs() @ B.double().abs()
    rel = ((Cd.cpu().double() - ref).abs() / mag).max().item()
    Ct = A.to(dev) @ B.to(dev)
    rel_t = ((Ct.cpu().double() - ref).abs() / mag).max().item()
    _say(f"gemm wide dynamic range: max error / sum|a||b| = {rel:.2e} (torch fp32: {rel_t:.2e})")
    assert rel < 2e-6, rel


def test_gemm_f32_tri_and_ktrim(dev):
    n = 384
    A = _rand((n, 128), 4)
    C0 = _rand((n, n), 5)
    Cd = C0.clone().to(dev)
    Ad = A.to(dev)
    # upper block triangle only: C -= A A^T
    ops.gemm_f32_(Ad, 128, 1, Ad, 1, 128, Cd, n, n, 128, alpha=-1.0, beta=1.0, tri=1)
    ref = C0.double() - A.double() @ A.double().t()
    out = Cd.cpu().double()
    for bi in range(3):
        for bj in range(3):
            blk = (slice(bi * 128, bi * 128 + 128), slice(bj * 128, bj * 128 + 128))
            want = ref[blk] if bi <= bj else C0.double()[blk]
            assert (out[blk] - want).abs().max().item() < 5e-3
    # ktrim=2: A upper triangular with garbage below the block diagonal
    T = torch.triu(_rand((n, n), 6))
    Tg = T.clone()
    for bi in range(3):
        for bj in range(bi):
            Tg[bi * 128:(bi + 1) * 128, bj * 128:(bj + 1) * 128] = float("nan")
    B = _rand((n, 200), 7)
    out = torch.zeros(n, 200, device=dev)
    ops.gemm_f32_(Tg.to(dev), n, 1, B.to(dev), 200, 1, out, n, 200, n, ktrim=2)
    assert (out.cpu().double() - T.double() @ B.double()).abs().max().item() < 5e-3
    # ktrim=1: A(m,k) = T[k,m]
    out = torch.zeros(n, 200, device=dev)
    ops.gemm_f32_(Tg.to(dev), 1, n, B.to(dev), 200, 1, out, n, 200, n, ktrim=1)
    assert (out.cpu().double() - T.double().t() @ B.double()).abs().max().item() < 5e-3


# ---------------------------------------------------------------- (1) Hessian SYRK
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("n,C", [(1024, 896), (4096, 256), (100, 128), (33, 384), (5000, 640)])
def test_hessian_syrk_vs_fp64(dev, n, C, dtype):
    """Every activation dtype the reference's driver offers (quant.py:79-81), against the fp64 closed form of the
    values as stored in that dtype: the 1e-5 relative Frobenius gate."""
    _say(f"syrk n={n} C={C} {dtype}")
    X = synth.activations_outlier(n, C, seed=n + C, dtype=dtype)
    H = torch.zeros(C, C, device=dev)
    ops.hessian_syrk_(H, X.to(dev), 0.0, 2.0 / n)
    H64 = O.hessian_fp64([X])
    Hc = H.cpu().double()
    assert ((Hc - H64).norm() / H64.norm()).item() < 1e-5  # the 1e-5 Frobenius gate
    assert torch.equal(Hc, Hc.t())  # mirrored exactly


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_hessian_running_mean_matches_oracle(dev, dtype):
    C = 512
    X = synth.activations_swiglu(3000, C, seed=9, dtype=dtype)
    chunks = [X[:700], X[700:701], X[701:2500], X[2500:]]
    H = torch.zeros(C, C, device=dev)
    Href, n = None, 0
    for x in chunks:
        beta, alpha = n / (n + x.shape[0]), 2.0 / (n + x.shape[0])
        ops.hessian_syrk_(H, x.to(dev), beta, alpha)
        Href, n = O.hessian_update(Href, n, x)
    H64 = O.hessian_fp64(chunks)
    assert ((H.cpu().double() - H64).norm() / H64.norm()).item() < 1e-5
    assert ((H.cpu() - Href).norm() / Href.norm()).item() < 1e-5


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("C,ns", [(512, [700, 300, 1500, 256, 4000]), (256, [300] * 18), (384, [100, 600, 0])])
def test_hessian_syrk_grouped(dev, C, ns, dtype):
    """Several Hessians in one call: each within the 1e-5 gate of fp64 and equal to the one-at-a-time result up to
    the order of the fp32 token sum."""
    _say(f"grouped syrk C={C} ns={ns} {dtype}")
    Xs = [synth.activations_outlier(n, C, seed=50 + i, dtype=dtype) for i, n in enumerate(ns)]
    H0 = [_rand((C, C), 70 + i) for i in range(len(ns))]
    H0 = [h + h.t() for h in H0]
    betas = [0.25 * (i % 3) for i in range(len(ns))]
    alphas = [2.0 / max(n, 1) for n in ns]
    Hg = [h.clone().to(dev) for h in H0]
    ops.hessian_syrk_grouped_(Hg, [x.to(dev) for x in Xs], betas, alphas, mirror=True)
    for i, n in enumerate(ns):
        ref = betas[i] * H0[i].double() + alphas[i] * (Xs[i].double().t() @ Xs[i].double())
        got = Hg[i].cpu().double()
        assert ((got - ref).norm() / ref.norm()).item() < 1e-5, (i, n)
        assert torch.equal(got, got.t())
        Hs = H0[i].clone().to(dev)
        ops.hessian_syrk_(Hs, Xs[i].to(dev), betas[i], alphas[i])
        assert ((Hs.cpu().double() - got).norm() / ref.norm()).item() < 1e-6


def test_hessian_upper_only(dev):
    C, n = 512, 512
    X = synth.activations_outlier(n, C, seed=3).to(dev)
    H = torch.full((C, C), 7.0, device=dev)
    ops.hessian_syrk_(H, X, 0.0, 1.0, mirror=False)
    Hc = H.cpu()
    ref = (X.cpu().double().t() @ X.cpu().double())
    assert (torch.triu(Hc).double() - torch.triu(ref)).abs().max() / ref.abs().max() < 1e-5
    assert torch.all(Hc[256:, :256] == 7.0)  # below the diagonal tiles nothing is written
    ops.symmetrize_upper_(H)
    Hc = H.cpu()
    assert torch.equal(Hc, Hc.t()) and (Hc.double() - ref).abs().max() / ref.abs().max() < 1e-5


# ---------------------------------------------------------------- (2) factorisation
def _spd(C, seed, n=None):
    X = synth.activations_outlier(n or (C + C // 8), C, seed)
    H, _ = O.hessian_update(None, 0, X)
    H.diagonal().add_(0.01 * H.diag().mean())
    return H


@pytest.mark.parametrize("C", [128, 256, 384, 640, 896, 1024, 1536, 2176, 2432])  # 1 .. 19 blocks: every phase of the panel batches
def test_factor_vs_torch_chain(dev, C):
    _say(f"factor C={C}")
    H = _spd(C, C)
    Hi = torch.cholesky_inverse(torch.linalg.cholesky(H.double()))
    U64 = torch.linalg.cholesky(Hi, upper=True)
    U64 = U64 / U64.diag()[:, None]
    A = H.clone().to(dev)
    info = ops.factor_upper_inverse_(A)
    assert int(info.item()) == 0
    U = A.cpu()
    assert torch.equal(torch.tril(U, -1), torch.zeros_like(U))
    assert torch.equal(U.diag(), torch.ones(C))
    rel = ((U.double() - U64).norm() / U64.norm()).item()
    # the fp32 torch chain itself sits at ~1e-6 from the fp64 answer
    Hi32 = torch.cholesky_inverse(torch.linalg.cholesky(H))
    U32 = torch.linalg.cholesky(Hi32, upper=True)
    U32 = U32 / U32.diag()[:, None]
    rel32 = ((U32.double() - U64).norm() / U64.norm()).item()
    _say(f"  rel err vs fp64: ours {rel:.2e}, torch fp32 chain {rel32:.2e}")
    assert rel < max(5e-6, 5 * rel32)


@pytest.mark.parametrize("C", [128, 256, 1024])
def test_factor_from_equals_in_place(dev, C):
    """The entry point that leaves H untouched builds the same bits as the in-place one, on a destination full of NaN."""
    _say(f"factor_from C={C}")
    H = torch.empty(C, C + 64, device=dev)[:, :C]  # a row pitch of its own
    H.copy_(_spd(C, seed=17))
    H0 = H.clone()
    A = H.clone()
    info_a = ops.factor_upper_inverse_(A)
    lib = __import__("moe_quant_amd._lib", fromlist=["load"]).load()
    U = torch.full((C, C), float("nan"), device=dev)
    info_u = torch.zeros(1, dtype=torch.int32, device=dev)
    rc = lib.mq_factor_upper_inverse_from(H.data_ptr(), H.stride(0), U.data_ptr(), U.stride(0), C, 1, info_u.data_ptr(),
                                          None)
    torch.cuda.synchronize()
    assert rc == 0 and int(info_a.item()) == 0 and int(info_u.item()) == 0
    assert torch.equal(H, H0)
    assert torch.equal(U, A)
    # H == A is refused
    assert lib.mq_factor_upper_inverse_from(H.data_ptr(), C, H.data_ptr(), C, C, 1, info_u.data_ptr(), None) != 0


def test_factor_full_width_on_concurrent_streams(dev):
    """C = 7168 (56 block steps, launches of more workgroups than the chip holds at once), four factorisations
    in flight on four streams, twice: every result has the same bits, and U H U^T is diagonal.  The in-place
    panel product must not let one workgroup overwrite rows another still reads: a tiling that did passed every
    small case and lost a sixth of the codes at this size under load."""
    C = 7168
    _say(f"factor C={C} on four streams")
    gen = torch.Generator(device=dev).manual_seed(91)
    X = torch.randn(8192, C, generator=gen, device=dev)
    H = (X.t() @ X) / 8192
    del X
    H.diagonal().add_(0.01 * H.diag().mean())
    lanes = [torch.cuda.Stream(device=dev) for _ in range(4)]
    outs = []
    for rep in range(2):
        for ln in lanes:
            ln.wait_stream(torch.cuda.current_stream(dev))
            with torch.cuda.stream(ln):
                U, info = ops.factor_upper_inverse_from(H)
                outs.append((U, info))
    torch.cuda.synchronize()
    for U, info in outs:
        assert int(info.item()) == 0
        assert torch.equal(U, outs[0][0])
    U = outs[0][0]
    del outs
    T = U @ H @ U.t()
    d = T.diagonal().clone()
    T.diagonal().zero_()
    rel = (T.norm() / d.norm()).item()
    _say(f"  off-diagonal of U H U^T relative to its diagonal: {rel:.2e}")
    assert rel < 1e-4


def test_factor_reports_non_pd(dev):
    C = 256
    H = _spd(C, 77)
    H[200, 200] = -1.0
    A = H.to(dev)
    info = ops.factor_upper_inverse_(A)
    assert int(info.item()) == 201
    assert torch.equal(A.cpu(), torch.eye(C))  # the fallback GPTQ takes when Cholesky raises, src/gptq.py:239-240
    H = _spd(C, 78)
    H[5, 9] = float("nan")
    info = ops.factor_upper_inverse_(H.to(dev))
    assert int(info.item()) != 0


# ---------------------------------------------------------------- Hessian hygiene (src/gptq.py:140-146, 221-234)
def _prestep_reference(H):
    """The torch statements of quantization_pre_step on a full matrix."""
    H = H.clone()
    nan = bool(torch.isnan(H).any())
    if nan:
        H = torch.eye(H.shape[0])
    pruned = torch.diag(H) == 0
    H[pruned, pruned] = 1
    return H, pruned, nan


@pytest.mark.parametrize("C", [64, 200, 448])
@pytest.mark.parametrize("upper_only", [True, False])
def test_hessian_prestep(dev, C, upper_only):
    _say(f"prestep C={C} upper_only={upper_only}")
    X = _rand((3 * C, C), 11 + C)
    X[:, [5, C - 1]] = 0  # two input channels that never fire
    H = X.t() @ X / X.shape[0]
    H = torch.triu(H) + torch.triu(H, 1).t()  # exactly symmetric
    ref, pruned_ref, _ = _prestep_reference(H)
    Hd = (torch.triu(H) + torch.tril(torch.full_like(H, 7.0), -1)) if upper_only else H.clone()
    Hd = Hd.to(dev)
    pruned, flags = ops.hessian_prestep_(Hd, upper_only)
    assert torch.equal(Hd.cpu(), ref)
    assert torch.equal(pruned.cpu().bool(), pruned_ref)
    assert flags.cpu().tolist()[:2] == [0, 2]


@pytest.mark.parametrize("where", ["upper", "diag", "lower"])
def test_hessian_prestep_nan_gives_identity(dev, where):
    C = 192
    H = _spd(C, 3)
    r, c = {"upper": (10, 150), "diag": (70, 70), "lower": (150, 10)}[where]
    H[r, c] = float("nan")
    Hd = H.to(dev)
    pruned, flags = ops.hessian_prestep_(Hd, False)
    assert flags[0].item() != 0 and flags[1].item() == 0
    assert torch.equal(Hd.cpu(), torch.eye(C)) and not pruned.any().item()
    if where != "lower":  # with upper_only the lower triangle is never read
        Hd = H.to(dev)
        pruned, flags = ops.hessian_prestep_(Hd, True)
        assert flags[0].item() != 0 and torch.equal(Hd.cpu(), torch.eye(C))


@pytest.mark.parametrize("R,C,dtype", [(96, 256, torch.bfloat16), (50, 200, torch.bfloat16), (33, 130, torch.float32),
                                       (64, 136, torch.float16)])
def test_hessian_damp(dev, R, C, dtype):
    _say(f"damp R={R} C={C} {dtype}")
    H = _spd(C, 21 + C)
    W = _rand((R, C), 5, 0.02).to(dtype)
    W[:, [3, C - 2]] = 0
    W[0, 3] = -0.0
    pruned = torch.zeros(C, dtype=torch.uint8)
    pruned[[9, 40]] = 1
    # torch statements of _get_hessian_inverse on the weights with pruned columns zeroed
    w = W.float().clone()
    w[:, pruned.bool()] = 0
    ref = H.clone()
    zero_cols = torch.nonzero(w.eq(0).all(dim=0))
    ref[zero_cols, :] = 0
    ref[:, zero_cols] = 0
    ref[zero_cols, zero_cols] = 1
    damp = 0.01 * torch.diag(ref).mean()
    ref[range(C), range(C)] += damp
    Hd = H.to(dev)
    flags = torch.zeros(4, dtype=torch.int32, device=dev)
    ops.hessian_damp_(Hd, W.to(dev), pruned.to(dev), 0.01, flags)
    out = Hd.cpu()
    assert flags[2].item() == 4
    off = ~torch.eye(C, dtype=torch.bool)
    assert torch.equal(out[off], ref[off])
    # the mean runs in another order than torch's: the damping term may differ in its last bits
    assert torch.allclose(out.diag(), ref.diag(), rtol=1e-6, atol=0)
    # no dead channel: only the diagonal moves
    Hd = H.to(dev)
    ops.hessian_damp_(Hd, torch.ones(R, C, dtype=dtype, device=dev), None, 0.05, flags)
    assert flags[2].item() == 0
    ref2 = H.clone()
    ref2[range(C), range(C)] += 0.05 * torch.diag(H).mean()
    assert torch.equal(Hd.cpu()[off], H[off]) and torch.allclose(Hd.cpu().diag(), ref2.diag(), rtol=1e-6, atol=0)


def test_inv_sym(dev):
    from moe_quant_amd.linalg_utils import inv_sym

    for C in (200, 384):
        H = _spd(C, 5 + C)
        Hi = inv_sym(H.to(dev)).cpu().double()
        ref = torch.linalg.inv(H.double())
        assert ((Hi - ref).norm() / ref.norm()).item() < 1e-4
    with pytest.raises(torch.linalg.LinAlgError):
        inv_sym(-torch.eye(128, device=dev))


# ---------------------------------------------------------------- (3) grid / layout / loop
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("g", [32, 128, 384])
def test_grid_bit_exact(dev, dtype, g):
    R, C = 96, 768
    W = (_rand((R, C), 11, 0.02)).to(dtype)
    W[3, 128:256] = 0  # all-zero group -> bf16(1e-12)
    rd = torch.bfloat16 if dtype == torch.float32 else dtype
    s_ref, z_ref, maxq = O.quantization_grid(W.float(), g, 4, rd)
    s_rg, s_gr = ops.quant_grid_sym(W.to(dev), g, 4, rd)
    assert torch.equal(s_rg.cpu(), s_ref)
    assert torch.equal(s_gr.cpu(), s_ref.t())


@pytest.mark.parametrize("g", [32, 128, 512])
def test_grid_wide_rows_and_dead_columns(dev, g):
    """Rows wider than one wavefront pass of the 16-byte kernel (2048 columns), ragged last pass, dead columns."""
    R, C = 40, 2048 + 1536
    W = _rand((R, C), 21, 0.02).bfloat16()
    dead = torch.zeros(C, dtype=torch.uint8)
    dead[[0, 5, 2047, 2048, C - 1]] = 1
    dead[1024:1024 + g] = 1  # a whole group dead -> bf16(1e-12)
    Wm = W.float().clone()
    Wm[:, dead.bool()] = 0
    s_ref, _, _ = O.quantization_grid(Wm, g, 4, torch.bfloat16)
    s_rg, s_gr = ops.quant_grid_sym(W.to(dev), g, 4, torch.bfloat16, dead_cols=dead.to(dev))
    assert torch.equal(s_rg.cpu(), s_ref)
    assert torch.equal(s_gr.cpu(), s_ref.t())


def test_prepare_and_untranspose(dev):
    R, C = 200, 320
    W = _rand((R, C), 12, 0.02).bfloat16()
    perm = torch.randperm(C, generator=torch.Generator().manual_seed(1))
    dead = torch.zeros(C, dtype=torch.uint8)
    dead[[3, 77]] = 1
    Wt = ops.prepare_wt(W.to(dev), perm.to(torch.int32).to(dev), dead.to(dev)).cpu()
    ref = W.float().clone()
    ref[:, dead.bool()] = 0
    assert torch.equal(Wt, ref.t()[perm])
    Q = torch.randint(0, 16, (C, R), dtype=torch.uint8)
    perm_inv = torch.argsort(perm)
    codes = ops.untranspose_codes(Q.to(dev), perm_inv.to(torch.int32).to(dev)).cpu()
    assert torch.equal(codes, Q[perm_inv].t())
    packed = ops.pack_from_qt(Q.to(dev), perm_inv.to(torch.int32).to(dev)).cpu()
    assert torch.equal(packed, O.pack_to_int32(codes.to(torch.int8) - 8, 4))


def _loop_case(R, C, seed, g=128, act_order=False):
    W = synth.weight(R, C, seed)
    X = synth.activations_outlier(C + C // 4, C, seed + 1)
    H, _ = O.hessian_update(None, 0, X)
    H, W32, _, _ = O.quantization_pre_step(H, W)
    s, z, maxq = O.quantization_grid(W32, g, 4, torch.bfloat16)
    s_rep, z_rep = O.replicate_grid(s, z, g)
    perm, perm_inv = O.act_order_perm(H, act_order)
    Hp = H[perm][:, perm]
    U, ok = O.hessian_inverse(Hp, W32, 0.01)
    return W32, U.contiguous(), s, s_rep, z_rep, maxq, perm, perm_inv


@pytest.mark.parametrize(
    "R,C,block,g", [(256, 512, 128, 128), (100, 384, 128, 128), (64, 300, 128, 100), (130, 256, 64, 128), (64, 128, 128, 128),
                    (64, 1024, 128, 128), (96, 900, 128, 100), (70, 1300, 128, 100)]  # 8+ blocks: the error ring wraps
)
def test_loop_vs_oracle_same_U(dev, R, C, block, g):
    _say(f"loop R={R} C={C} block={block} g={g}")
    W32, U, s, s_rep, z_rep, maxq, perm, _ = _loop_case(R, C, 31 + R, g=g)
    Wt_ref = W32.t()[perm].contiguous()
    q_ref = O.gptq_loop(Wt_ref, U, s_rep.t()[perm].contiguous(), z_rep.t()[perm].contiguous(), maxq,
                        torch.bfloat16, block)
    Wt = W32.t()[perm].contiguous().to(dev)
    st = s_rep.t()[perm].contiguous().to(dev)
    zt = z_rep.t()[perm].contiguous().to(dev)
    Qt = ops.gptq_loop_(Wt, U.to(dev), st, None, zt, 0.0, 15.0, torch.bfloat16, block)
    match = (Qt.cpu().float() == q_ref).float().mean().item()
    _say(f"  code match {match:.6f}")
    assert match >= 0.999
    # dequantized weights written back must equal (q - 8) * s exactly
    assert torch.equal(Wt.cpu(), ((Qt.cpu().float() - 8.0) * st.cpu()).bfloat16().float())


def test_loop_identity_U_is_round_to_nearest(dev):
    R, C = 128, 256
    W32, _, s, s_rep, z_rep, maxq, _, _ = _loop_case(R, C, 5)
    Wt = W32.t().contiguous().to(dev)
    st = s_rep.t().contiguous().to(dev)
    Qt = ops.gptq_loop_(Wt, torch.eye(C, device=dev), st, None, None, 8.0, 15.0, torch.bfloat16, 128)
    want = torch.floor(W32.t() / s_rep.t() + 8.5).clamp(0, 15)
    assert torch.equal(Qt.cpu().float(), want)


def test_loop_quantizer_arithmetic_is_ieee_exact(dev):
    """With U = I every column is quantized on its own: 2M (w, s) pairs, including tiny and huge ratios,
    must give exactly floor(w / s + 8.5) with IEEE division (the kernel hoists a reciprocal out of the chain)."""
    R, C = 2048, 1024
    g = torch.Generator().manual_seed(99)
    W = torch.randn(R, C, generator=g) * 0.02
    W[:, 100] = 0.0
    W[:, 101] *= 1e4
    W[:, 102] *= 1e-6
    W[5, :] = torch.linspace(-0.2, 0.2, C)
    s = (torch.rand(C, R, generator=g) * 0.02 + 1e-4).bfloat16().float()
    s[103] = torch.tensor(1e-12).bfloat16().float()  # the all-zero-group scale
    s[200:300] = (W.t()[200:300].abs() / 7.5 + 1e-12).bfloat16().float()  # values that land on .5 boundaries often
    Wt = W.t().contiguous()
    want = torch.floor(Wt / s + 8.0 + 0.5).clamp(0, 15)
    Wd = Wt.clone().to(dev)
    Qt = ops.gptq_loop_(Wd, torch.eye(C, device=dev), s.to(dev), None, None, 8.0, 15.0, torch.bfloat16, 128)
    assert torch.equal(Qt.cpu().float(), want)
    assert torch.equal(Wd.cpu(), ((want - 8.0) * s).bfloat16().float())


@pytest.mark.parametrize("rd", [torch.bfloat16, torch.float16, torch.float32])
def test_loop_block_wide_scale_row_is_ieee_exact(dev, rd):
    """Grouped scales whose group covers a whole block: the kernel divides through a reciprocal computed once per
    block (q0 = x*rcp, q1 = fma(fma(-q0, s, x), rcp, q0)).  With U = I, 2M (w, s) pairs incl. zero, tiny and huge
    scales must give exactly floor(w / s + 8.5) with IEEE division, and the dequantized weights the rounded (q-8)*s."""
    R, C, gsz = 2048, 1024, 128
    g = torch.Generator().manual_seed(123)
    W = torch.randn(R, C, generator=g) * 0.02
    W[:, 100] = 0.0
    W[5, :] = torch.linspace(-0.2, 0.2, C)
    G = C // gsz
    s = (torch.rand(G, R, generator=g) * 0.02 + 1e-4).bfloat16().float()
    s[1, :512] = torch.tensor(1e-12).bfloat16().float()   # the all-zero-group scale
    s[2, :512] = 0.0                                       # division by zero: +-inf and NaN quotients
    s[3, :512] = 3.0e-39                                   # a denormal scale: its reciprocal overflows
    s[4] = (W[:, 4 * gsz:5 * gsz].abs().amax(1) / 7.5 + 1e-12).bfloat16().float()  # many .5 boundaries
    s[5, :512] = 1e30                                      # tiny quotients
    srow = (torch.arange(C) // gsz).to(torch.int32)
    Wt = W.t().contiguous()
    s_rep = s[srow.long()]                                 # (C, R)
    want = torch.floor(Wt / s_rep + 8.0 + 0.5)
    want = torch.where(torch.isnan(want), torch.zeros_like(want), want).clamp(0, 15)  # fmax(NaN, 0) = 0
    Wd = Wt.clone().to(dev)
    Qt = ops.gptq_loop_(Wd, torch.eye(C, device=dev), s.to(dev), srow.to(dev), None, 8.0, 15.0, rd, 128)
    assert torch.equal(Qt.cpu().float(), want)
    deq = ((want - 8.0) * s_rep).to(rd).float()
    got = Wd.cpu()
    ok = torch.isfinite(deq)
    assert torch.equal(got[ok], deq[ok])


def test_loop_compact_scale_and_perm(dev):
    R, C, g = 128, 512, 64
    W32, U, s, s_rep, z_rep, maxq, perm, perm_inv = _loop_case(R, C, 8, g=g, act_order=True)
    Wt_ref = W32.t()[perm].contiguous()
    q_ref = O.gptq_loop(Wt_ref, U, s_rep.t()[perm].contiguous(), z_rep.t()[perm].contiguous(), maxq,
                        torch.bfloat16, 128)
    Wt = ops.prepare_wt(W32.to(dev), perm.to(torch.int32).to(dev))
    scale_row = (perm // g).to(torch.int32).to(dev)
    Qt = ops.gptq_loop_(Wt, U.to(dev), s.t().contiguous().to(dev), scale_row, None, 8.0, 15.0, torch.bfloat16, 128)
    assert (Qt.cpu().float() == q_ref).float().mean().item() >= 0.999


# ---------------------------------------------------------------- (4) packer
@pytest.mark.parametrize("R,C", [(64, 128), (7, 24), (33, 100), (5, 7), (1, 8), (256, 2048)])
def test_pack_bit_exact(dev, R, C):
    q = torch.randint(0, 16, (R, C), dtype=torch.uint8, generator=torch.Generator().manual_seed(R * C))
    want = O.pack_to_int32(q.to(torch.int8) - 8, 4)
    got = ops.pack_int4(q.to(dev)).cpu()
    assert torch.equal(got, want)
    # explicit zero points (the general form pack_weight uses)
    g = C if C % 8 else 8
    zero = torch.full((R, C // g), 8.0)
    got = ops.pack_int4(q.to(dev), zero.to(dev), g).cpu()
    assert torch.equal(got, want)
    # round trip
    assert torch.equal(O.unpack_from_int32(got, 4, (R, C)) + 8, q.to(torch.int8))


# ---------------------------------------------------------------- scale search (src/quant_utils.py:104-192)
@pytest.mark.parametrize("R,C,g,dtype", [(256, 512, 128, torch.bfloat16), (64, 384, 64, torch.bfloat16),
                                         (40, 200, 100, torch.float32), (32, 256, 32, torch.float16)])
def test_mse_scale_search(dev, R, C, g, dtype):
    """Scales after the search equal the oracle's except where two candidates' losses tie to within the rounding of
    log/exp (the kernel uses the hardware's base-2 pair, the oracle torch's natural ones): there the chosen
    candidate must still be as good as the oracle's."""
    _say(f"mse scale R={R} C={C} g={g} {dtype}")
    W = synth.weight(R, C, 11 + R, dtype=dtype)
    W[:, ::37] *= 3.0  # outliers, so that shrinking pays off in many groups
    W[3, g : 2 * g] = 0  # an all-zero group: every loss is 0, the last candidate wins
    p = O.search_points()
    x = W.float().reshape(R, C // g, g)
    rd = dtype if dtype != torch.float32 else torch.bfloat16
    s0, z0, maxq = O.find_quantization_meta(x, 4, rd)
    want = O.mse_scale(x.contiguous(), p, s0, z0, maxq, rd, 2.4)
    s_rg, s_gr = ops.quant_grid_sym(W.to(dev), g, 4, rd)
    assert torch.equal(s_rg.cpu(), s0)
    ops.mse_scale_sym_(W.to(dev), g, p.to(dev), s_rg, s_gr, 8.0, 15.0, 2.4, rd)
    got = s_rg.cpu()
    assert torch.equal(s_gr.cpu(), got.t())
    same = (got == want).float().mean().item()
    _say(f"  scales equal to the oracle's: {same:.4f}; moved by the search: {(want != s0).float().mean().item():.3f}")
    assert same >= 0.97
    assert torch.equal(got[3, 1], (s0[3, 1] * p[-1]).to(rd).float())

    def loss(sc):
        q = torch.floor(x / sc[..., None] + 8.5).clamp(0, 15)
        dq = ((q - 8.0) * sc[..., None]).to(rd).float()
        return (dq - x).abs().double().pow(2.4).sum(-1)

    lg, lw = loss(got), loss(want)
    ok = ~torch.isnan(lw)  # fp16 rounds the 1e-12 scale of the all-zero group to 0: 0/0 there
    assert torch.all(lg[ok] <= lw[ok] * (1 + 1e-4) + 1e-30)


# ---------------------------------------------------------------- FP8 checkpoint ingest (src/quant_utils.py:267-298)
@pytest.mark.parametrize("R,C", [(256, 512), (130, 260), (7, 33), (2048, 7168)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fp8_block_dequant_bit_exact(dev, R, C, dtype):
    from moe_quant_amd import quant_utils

    _say(f"fp8 dequant {R}x{C} {dtype}")
    g = torch.Generator().manual_seed(R + C)
    W8 = torch.randint(0, 256, (R, C), generator=g, dtype=torch.uint8)
    W8[0, : min(C, 256)] = torch.arange(min(C, 256), dtype=torch.uint8)  # every byte value, NaNs included
    W8 = W8.view(torch.float8_e4m3fn)
    s = torch.rand((R + 127) // 128, (C + 127) // 128, generator=g) * 0.01 + 1e-4
    want = O.dequantize_fp8_entry(W8, s, dtype)
    got = ops.dequant_fp8_block(W8.to(dev), s.to(dev), dtype).cpu()
    assert got.dtype == dtype
    assert torch.equal(torch.nan_to_num(got.float(), nan=-77.0), torch.nan_to_num(want.float(), nan=-77.0))
    sd = {"a.weight": W8.to(dev), "a.weight_scale_inv": s.to(dev), "b.weight": torch.ones(2, 2, device=dev)}
    assert quant_utils.can_dequantize_from_fp8(sd)
    quant_utils.dequantize_state_dict(sd, dtype)
    assert set(sd) == {"a.weight", "b.weight"}
    assert torch.equal(torch.nan_to_num(sd["a.weight"].float().cpu(), nan=-77.0), torch.nan_to_num(want.float(), nan=-77.0))


# ---------------------------------------------------------------- grouped entry points: same bits as one call per problem
@pytest.mark.parametrize("C,G", [(640, 5), (256, 18), (128, 3), (1152, 2)])
def test_factor_grouped_equals_single_calls(dev, C, G):
    _say(f"grouped factor C={C} G={G}")
    Hs = [_spd(C, 900 + i).to(dev) for i in range(G)]
    bad = G // 2
    Hs[bad] = torch.eye(C, device=dev)
    Hs[bad][3, 70] = Hs[bad][70, 3] = 4.0  # not positive definite: identity fallback for this one only
    keep = [h.clone() for h in Hs]
    Us, infos = ops.factor_upper_inverse_from_grouped(Hs)
    infos = infos.cpu().tolist()
    for i in range(G):
        assert torch.equal(Hs[i], keep[i])  # inputs untouched
        U1, info1 = ops.factor_upper_inverse_from(keep[i])
        assert torch.equal(Us[i], U1), i
        assert infos[i] == int(info1.item()) and (infos[i] != 0) == (i == bad)
    assert torch.equal(Us[bad], torch.eye(C, device=dev))


@pytest.mark.parametrize("C,R,G,order", [(512, 192, 3, False), (384, 300, 17, True), (256, 64, 2, False)])
def test_loop_grouped_equals_single_calls(dev, C, R, G, order):
    _say(f"grouped loop C={C} R={R} G={G} permuted={order}")
    g = 128
    Wts, Us, scs, maps = [], [], [], []
    for i in range(G):
        W = synth.weight(R, C, 700 + i).to(dev)
        U, _ = ops.factor_upper_inverse_from(_spd(C, 800 + i).to(dev))
        perm = torch.randperm(C, generator=torch.Generator().manual_seed(i)).to(dev) if order else torch.arange(C, device=dev)
        s_rg, s_gr = ops.quant_grid_sym(W, g, 4, torch.bfloat16)
        Wts.append(ops.prepare_wt(W, perm.to(torch.int32)))
        Us.append(U)
        scs.append(s_gr)
        maps.append((perm // g).to(torch.int32))
    singles = []
    for i in range(G):
        w = Wts[i].clone()
        q = ops.gptq_loop_(w, Us[i], scs[i], maps[i], None, 8.0, 15.0, torch.bfloat16, 128)
        singles.append((w, q))
    Qts = ops.gptq_loop_grouped_(Wts, Us, scs, maps, 8.0, 15.0, torch.bfloat16, 128)
    for i in range(G):
        assert torch.equal(Qts[i], singles[i][1]), i
        assert torch.equal(Wts[i], singles[i][0]), i


# ---------------------------------------------------------------- the loop's inverse-free form: Cholesky multipliers
def _rev_chol64(H):
    """R upper with H = R R^T, in fp64 (Cholesky of the index-reversed matrix)."""
    C = H.shape[0]
    J = torch.arange(C - 1, -1, -1)
    L = torch.linalg.cholesky(H.double()[J][:, J])
    return L[J][:, J]


@pytest.mark.parametrize("C", [128, 256, 384, 640, 1024, 2176])
def test_factor_chol_vs_fp64(dev, C):
    """F[j,k] = -R[j,k]/R[k,k] above the diagonal against an fp64 reverse Cholesky, and the identity it rests on:
    F equals -(U^-1)[j,k]-type multipliers of the classical factor, i.e. (I - F_strict) is the inverse of the
    unit-diagonal U's column-normalised form -- checked directly as  R = U^-1."""
    _say(f"chol factor C={C}")
    H = _spd(C, C + 7)
    R = _rev_chol64(H)
    want = torch.triu(-(R / R.diag()[None, :]), 1)
    F, info = ops.factor_chol(H.to(dev))
    assert int(info.item()) == 0
    got = torch.triu(F.cpu().double(), 1)
    rel = ((got - want).norm() / want.norm()).item()
    _say(f"  rel err vs fp64 {rel:.2e}")
    assert rel < 5e-6
    # against the classical factor of the same matrix: U = R^-1 row-normalised  =>  U_unnormalised * R = I
    U, _ = ops.factor_upper_inverse_from(H.to(dev), normalize=False)
    assert ((U.cpu().double() @ R) - torch.eye(C, dtype=torch.float64)).abs().max().item() < 5e-3


def test_factor_chol_grouped_and_failure(dev):
    C, G = 512, 5
    Hs = [_spd(C, 300 + i).to(dev) for i in range(G)]
    Hs[2] = torch.eye(C, device=dev)
    Hs[2][5, 300] = Hs[2][300, 5] = 3.0  # not positive definite
    keep = [h.clone() for h in Hs]
    Fs, infos = ops.factor_chol_grouped(Hs)
    infos = infos.cpu().tolist()
    for i in range(G):
        assert torch.equal(Hs[i], keep[i])
        F1, info1 = ops.factor_chol(keep[i])
        assert torch.equal(torch.triu(Fs[i], 1), torch.triu(F1, 1)), i
        assert infos[i] == int(info1.item()) and (infos[i] != 0) == (i == 2)
    assert torch.equal(torch.triu(Fs[2], 1), torch.zeros(C, C, device=dev))  # identity fallback: no propagation


@pytest.mark.parametrize("C,R,order", [(512, 256, False), (896, 192, True), (300, 70, False)])
def test_loop_chol_matches_classical_loop(dev, C, R, order):
    """The inverse-free loop (F, original weights) against the classical loop (U, quantization errors) on the same
    problem: the two are the same recurrence, so codes agree up to fp32 rounding; grouped calls equal single ones."""
    _say(f"chol loop C={C} R={R} permuted={order}")
    g = 128 if C % 128 == 0 else C
    Cp = (C + 127) // 128 * 128
    Hs, Ws = [], []
    for i in range(3):
        H = _spd(C, 500 + i)
        Hp = torch.eye(Cp)
        Hp[:C, :C] = H
        Hs.append(Hp.to(dev))
        Ws.append(synth.weight(R, C, 600 + i).to(dev))
    Fs, _ = ops.factor_chol_grouped(Hs)
    outs = []
    for i in range(3):
        U, _ = ops.factor_upper_inverse_from(Hs[i])
        perm = torch.randperm(C, generator=torch.Generator().manual_seed(i)).to(dev) if order else torch.arange(C, device=dev)
        s_rg, s_gr = ops.quant_grid_sym(Ws[i], g, 4, torch.bfloat16)
        srow = (perm // g).to(torch.int32)
        Wt = ops.prepare_wt(Ws[i], perm.to(torch.int32))
        q_u = ops.gptq_loop_(Wt, U, s_gr, srow, None, 8.0, 15.0, torch.bfloat16, 128)
        Wt2, W0t = ops.prepare_wt_pair(Ws[i], perm.to(torch.int32))
        assert torch.equal(Wt2, W0t)
        q_f = ops.gptq_loop_chol_grouped_([Wt2], [W0t], [Fs[i]], [s_gr], [srow], 8.0, 15.0, torch.bfloat16, 128)[0]
        same = (q_u == q_f).float().mean().item()
        _say(f"  problem {i}: codes equal {same:.6f}")
        assert same >= 0.999
        assert torch.equal(W0t, ops.prepare_wt(Ws[i], perm.to(torch.int32)))  # the original copy is untouched
        # dequantized weights out: Wt2 = (q - 8) * scale of the column's group, rounded to bf16
        sc_col = s_gr[srow.long()]  # (C, R)
        assert torch.equal(Wt2, ((q_f.float() - 8.0) * sc_col).to(torch.bfloat16).float())
        outs.append((Wt2, q_f, perm, s_gr, srow))
    pairs = [ops.prepare_wt_pair(Ws[i], outs[i][2].to(torch.int32)) for i in range(3)]
    Qg = ops.gptq_loop_chol_grouped_([p[0] for p in pairs], [p[1] for p in pairs], Fs, [o[3] for o in outs],
                                     [o[4] for o in outs], 8.0, 15.0, torch.bfloat16, 128)
    for i in range(3):
        assert torch.equal(Qg[i], outs[i][1]) and torch.equal(pairs[i][0], outs[i][0])


def test_loop_chol_on_a_rank_deficient_damped_hessian(dev):
    """Fewer tokens than input channels (n = C/8, as the lightly loaded experts of a MoE layer have): H is singular and
    held up by its 1% damping alone, the worst case for the inverse-free loop, whose columns hand on their total change
    z = y - w_original (a difference of larger terms than the classical loop's quantization error).  At real width, on
    the same damped matrix: the inverse-free loop (F) against the classical loop (U) and both against the CPU oracle's
    classical loop on its own fp32 factor of that matrix.  The bounds are measured floors minus a margin."""
    C, R, n = 7168, 256, 896
    X = synth.activations_outlier(n, C, 77).to(dev)
    W = synth.weight(R, C, 78)
    H = torch.zeros(C, C, device=dev)
    ops.hessian_syrk_(H, X, 0.0, 2.0 / n)
    H.diagonal().add_(0.01 * H.diagonal().mean())
    s_rg, s_gr = ops.quant_grid_sym(W.to(dev), 128, 4, torch.bfloat16)
    srow = (torch.arange(C, device=dev) // 128).to(torch.int32)
    U, _ = ops.factor_upper_inverse_from(H)
    F, info = ops.factor_chol(H)
    assert int(info.item()) == 0
    Wt = ops.prepare_wt(W.to(dev))
    q_u = ops.gptq_loop_(Wt, U, s_gr, srow, None, 8.0, 15.0, torch.bfloat16, 128)
    Wt2, W0t = ops.prepare_wt_pair(W.to(dev))
    q_f = ops.gptq_loop_chol_grouped_([Wt2], [W0t], [F], [s_gr], [srow], 8.0, 15.0, torch.bfloat16, 128)[0]
    Hc = H.cpu()
    Uc = torch.linalg.cholesky(torch.cholesky_inverse(torch.linalg.cholesky(Hc)), upper=True)
    Uc = Uc / Uc.diag()[:, None]
    sc, zz, maxq = O.quantization_grid(W.float(), 128, 4, torch.bfloat16)
    sr, zr = O.replicate_grid(sc, zz, 128)
    q_o = O.gptq_loop(W.float().t().contiguous(), Uc, sr.t().contiguous(), zr.t().contiguous(), maxq, torch.bfloat16, 128)
    m_fu = (q_f == q_u).float().mean().item()
    m_fo = (q_f.cpu().float() == q_o).float().mean().item()
    m_uo = (q_u.cpu().float() == q_o).float().mean().item()
    _say(f"rank-deficient H (n={n}, C={C}): chol loop vs U loop {m_fu:.5f}; chol loop vs oracle {m_fo:.5f}; "
         f"U loop vs oracle {m_uo:.5f}")
    # measured: 0.9993 between the two HIP forms, 0.9945 for either against the oracle (two fp32 factorisations of a
    # matrix whose smallest eigenvalues are the damping term differ more than two walks over the same factorisation)
    assert m_fu >= 0.998 and m_fo >= 0.99 and m_uo >= 0.99
    assert m_fo >= m_uo - 0.002  # the inverse-free form loses nothing against the classical one


@pytest.mark.parametrize("C", [128, 1000, 7168, 18432])
def test_permute_symmetric_equals_torch_gather(dev, C):
    """Act-order gather (src/gptq.py:187): bit-identical to H[perm][:, perm], input untouched."""
    g = torch.Generator(device=dev).manual_seed(C)
    H = torch.randn(C, C, generator=g, device=dev)
    perm = torch.argsort(H.diag(), descending=True)
    keep = H.clone() if C <= 7168 else None
    Hp = ops.permute_symmetric(H, perm.to(torch.int32))
    assert torch.equal(Hp, H[perm][:, perm])
    if keep is not None:
        assert torch.equal(H, keep)


def test_hessian_syrk_tail_round_split(dev):
    """7168 channels are 406 tiles of 256x256 on 256 CUs: from 32768 tokens on the 150 tiles of the last round are cut
    into token ranges whose partial sums meet in the workspace.  Against an fp64 product formed on the GPU, with a
    ragged token count, accumulating onto an old H."""
    from moe_quant_amd import _lib

    C, n = 7168, 32768 + 40
    assert _lib.load().mq_hessian_syrk_workspace_bytes(n, C) > 0
    g = torch.Generator(device=dev).manual_seed(5)
    X = torch.randn(n, C, generator=g, device=dev)
    X[:, synth.outlier_channels(C, 6).to(dev)] *= 20.0
    X = X.to(torch.bfloat16)
    H0 = torch.randn(C, C, generator=g, device=dev)
    H0 = H0 + H0.t()
    H = H0.clone()
    ops.hessian_syrk_(H, X, 0.5, 2.0 / n, mirror=True)
    ref = torch.zeros(C, C, device=dev, dtype=torch.float64)
    for s0 in range(0, n, 8192):
        blk = X[s0:s0 + 8192].double()
        ref.addmm_(blk.t(), blk)
    ref = 0.5 * H0.double() + (2.0 / n) * ref
    err = ((H.double() - ref).norm() / ref.norm()).item()
    _say(f"tail-split syrk rel err {err:.2e}")
    assert err < 1e-5 and torch.equal(H, H.t())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,I", [(1, 8), (37, 2048), (700, 512), (0, 64)])
def test_swiglu_against_the_torch_expression(dev, n, I, dtype):
    """silu(g) * u as the chained torch ops compute it on 16-bit tensors (each op rounds its result): equal up to one
    unit in the last place of the 16-bit result (the exponential inside silu differs in its last fp32 bits)."""
    g = torch.Generator(device=dev).manual_seed(n + I)
    GU = (torch.randn(n, 2 * I, generator=g, device=dev) * 3).to(dtype)
    got = ops.swiglu(GU)
    want = torch.nn.functional.silu(GU[:, :I]) * GU[:, I:]
    assert got.shape == want.shape and got.dtype == dtype
    if n:
        ulp = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)
        assert ((got.float() - want.float()).abs() <= ulp * want.float().abs() + 1e-30).all()
        assert (got == want).float().mean().item() > 0.99


# ---------------------------------------------------------------- packed tokens: gather + re-layout, Hessian, SiLU product
@pytest.mark.parametrize("n,C", [(1, 8), (37, 264), (300, 512), (1000, 2048)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_pack_tokens_layout_and_gather(dev, n, C, dtype):
    """Xp[o][c][j] = X[rows[8 o + j]][c], zeros in the padding (tokens to a multiple of 128, channels to a multiple of
    256); the token-major copy written by the same pass equals X[rows]."""
    g = torch.Generator(device=dev).manual_seed(n + C)
    X = torch.randn(3 * n + 5, C, generator=g, device=dev).to(dtype)
    rows = torch.randint(0, X.shape[0], (n,), generator=g, device=dev)
    P, Xg = ops.pack_tokens(X, rows, also_token_major=True)
    assert torch.equal(Xg, X[rows]) and (P.n, P.C, P.dtype) == (n, C, dtype)
    Cp, npad = (C + 255) // 256 * 256, (n + 127) // 128 * 128
    full = P.data[: npad * Cp].view(npad // 8, Cp, 8).permute(0, 2, 1).reshape(npad, Cp)
    want = torch.zeros(npad, Cp, dtype=dtype, device=dev)
    want[:n, :C] = X[rows]
    assert torch.equal(full, want)
    assert torch.equal(ops.unpack_tokens(P), X[rows])
    P2 = ops.pack_tokens(X)  # no gather
    assert torch.equal(ops.unpack_tokens(P2), X)


@pytest.mark.parametrize("n,C,beta", [(300, 264, 0.0), (4096, 2048, 0.5), (32768 + 40, 7168, 0.25), (1, 512, 0.0),
                                      (9000, 1536, 1.0)])
def test_hessian_syrk_packed_vs_fp64(dev, n, C, beta):
    """The Hessian product on packed tokens against an fp64 product formed on the GPU (1e-5 relative Frobenius, the
    Hessian gate): few tiles cut into token ranges (C = 2048, 1536, 512), the tail-round split (7168 channels from 32768
    tokens on), padded channels (264), a single token, accumulation onto an old H."""
    g = torch.Generator(device=dev).manual_seed(n)
    X = torch.randn(n, C, generator=g, device=dev)
    X[:, synth.outlier_channels(C, 7).to(dev)] *= 20.0
    X = X.to(torch.bfloat16)
    H0 = torch.randn(C, C, generator=g, device=dev)
    H0 = H0 + H0.t()
    H = H0.clone()
    ops.hessian_syrk_packed_(H, ops.pack_tokens(X), beta, 2.0 / n, mirror=True)
    ref = torch.zeros(C, C, device=dev, dtype=torch.float64)
    for s0 in range(0, n, 8192):
        blk = X[s0:s0 + 8192].double()
        ref.addmm_(blk.t(), blk)
    ref = beta * H0.double() + (2.0 / n) * ref
    err = ((H.double() - ref).norm() / ref.norm()).item()
    _say(f"packed syrk n={n} C={C}: rel err {err:.2e}")
    assert err < 1e-5 and torch.equal(H, H.t())


@pytest.mark.parametrize("n,C", [(512, 520), (4100, 4104)])
def test_hessian_syrk_into_a_view_with_odd_pitch(dev, n, C):
    """H as a view into a larger buffer: rows 4 bytes off a 16-byte boundary and a pitch that is no multiple of four
    floats, so the kernels take their element-wise stores; same bits as into a plain matrix, nothing written outside."""
    _say(f"syrk into a strided view n={n} C={C}")
    g = torch.Generator(device=dev).manual_seed(n + C)
    X = torch.randn(n, C, generator=g, device=dev).bfloat16()
    plain = torch.full((C, C), 0.25, device=dev)
    ops.hessian_syrk_(plain, X, 0.5, 2.0 / n, mirror=True)
    big = torch.full((C + 2, C + 3), 0.25, device=dev)
    view = big[1 : C + 1, 2 : C + 2]
    assert view.data_ptr() % 16 != 0 and view.stride(0) % 4 != 0
    ops.hessian_syrk_(view, X, 0.5, 2.0 / n, mirror=True)
    assert torch.equal(view, plain)
    frame = big.clone()
    frame[1 : C + 1, 2 : C + 2] = 0.25
    assert torch.equal(frame, torch.full_like(big, 0.25))
    P = ops.pack_tokens(X)
    big.fill_(0.25)
    ops.hessian_syrk_packed_(view, P, 0.5, 2.0 / n, mirror=True)
    assert torch.equal(view, plain) or (view - plain).abs().max().item() <= 1e-6 * plain.abs().max().item()
    frame = big.clone()
    frame[1 : C + 1, 2 : C + 2] = 0.25
    assert torch.equal(frame, torch.full_like(big, 0.25))


def test_hessian_syrk_packed_grouped_and_fp16(dev):
    """Several Hessians of one width in one call, token counts far apart (a MoE layer's experts), fp16 tokens: each
    against its own fp64 product, and the handle API (update / update_many on PackedTokens) against plain tensors."""
    from moe_quant_amd.gptq import GPTQ

    C = 768
    ns = [256, 5000, 129, 2048 + 3]
    g = torch.Generator(device=dev).manual_seed(3)
    Xs = [torch.randn(n, C, generator=g, device=dev).to(torch.float16) for n in ns]
    Hs = [torch.zeros(C, C, device=dev) for _ in ns]
    ops.hessian_syrk_packed_grouped_(Hs, [ops.pack_tokens(X) for X in Xs], [0.0] * 4, [2.0 / n for n in ns], mirror=True)
    for H, X, n in zip(Hs, Xs, ns):
        ref = (2.0 / n) * (X.double().t() @ X.double())
        assert ((H.double() - ref).norm() / ref.norm()).item() < 1e-5
    lin = lambda: torch.nn.Linear(C, 64, bias=False, dtype=torch.float16, device=dev)
    a, b = [GPTQ(lin(), 128, True) for _ in ns], [GPTQ(lin(), 128, True) for _ in ns]
    GPTQ.update_many(a, [ops.pack_tokens(X) for X in Xs])
    GPTQ.update_many(a, [ops.pack_tokens(X[:200]) for X in Xs])
    a[0].update(ops.pack_tokens(Xs[0][:77]))
    GPTQ.update_many(b, Xs)
    GPTQ.update_many(b, [X[:200] for X in Xs])
    b[0].update(Xs[0][:77])
    for ha, hb in zip(a, b):
        assert ha.num_samples == hb.num_samples
        ha.symmetrize_hessian(), hb.symmetrize_hessian()
        assert ((ha.H - hb.H).norm() / hb.H.norm()).item() < 2e-6


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,I", [(1, 8), (37, 2048), (700, 520), (0, 64)])
def test_swiglu_packed_equals_swiglu(dev, n, I, dtype):
    """The SiLU product written in the packed layout holds the same bits as the token-major kernel's output; gate and
    up outputs given as the two halves of one stacked matrix (strided rows) or as two matrices."""
    g = torch.Generator(device=dev).manual_seed(n + I)
    GU = (torch.randn(n, 2 * I, generator=g, device=dev) * 3).to(dtype)
    want = ops.swiglu(GU)
    for G, U in ((GU[:, :I], GU[:, I:]), (GU[:, :I].contiguous(), GU[:, I:].contiguous())):
        P = ops.swiglu_packed(G, U)
        assert (P.n, P.C) == (n, I)
        if n:
            assert torch.equal(ops.unpack_tokens(P), want)
            Ip, npad = (I + 255) // 256 * 256, (n + 127) // 128 * 128
            full = P.data[: npad * Ip].view(npad // 8, Ip, 8).permute(0, 2, 1).reshape(npad, Ip)
            assert int((full[n:] != 0).sum()) == 0 and int((full[:, I:] != 0).sum()) == 0
