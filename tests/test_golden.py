"""The committed fixture against the oracle (CPU) and against the HIP path (GPU)."""
import os

import numpy as np
import pytest
import torch

from oracle import gptq_oracle as O

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tiny_gptq.npz"))


def _inputs():
    W = torch.from_numpy(G["W_bf16_bits"]).view(torch.bfloat16)
    X = torch.from_numpy(G["X_bf16_bits"]).view(torch.bfloat16)
    return W, X


def _check_H(H, tol):
    scale = np.abs(G["H_diag"]).max()
    assert np.abs(H.diag().numpy() - G["H_diag"]).max() <= tol * scale
    assert np.abs(H[[0, 100, 255]].numpy() - G["H_rows"]).max() <= tol * scale
    assert abs(H.double().norm().item() - float(G["H_fro"])) <= tol * float(G["H_fro"])


def test_oracle_reproduces_golden():
    torch.set_num_threads(1)
    W, X = _inputs()
    H, n = O.hessian_update(None, 0, X[:100])
    H, n = O.hessian_update(H, n, X[100:])
    _check_H(H, 1e-6)
    for tag, act in (("default", False), ("actorder", True)):
        r = O.quantize_linear(W, H.clone(), act_order=act)
        assert np.array_equal(r["perm"].numpy(), G[f"perm_{tag}"])
        assert np.array_equal(r["scale"].view(torch.int16).numpy(), G[f"scale_bits_{tag}"])
        assert (r["qweight"].numpy() == G[f"qweight_{tag}"]).mean() >= 0.999  # LAPACK builds may differ in the last bit
        packed = O.pack_to_int32(torch.from_numpy(G[f"qweight_{tag}"]).to(torch.int8) - 8, 4)
        assert np.array_equal(packed.numpy(), G[f"packed_{tag}"])


@pytest.mark.gpu
@pytest.mark.parametrize("tag,order", [("default", "default"), ("actorder", "activation")])
def test_hip_path_reproduces_golden(dev, tag, order):
    from moe_quant_amd.gptq import GPTQ
    from moe_quant_amd.pack_quantized_model import pack_weight

    W, X = _inputs()
    layer = torch.nn.Linear(W.shape[1], W.shape[0], bias=False, dtype=torch.bfloat16, device=dev)
    layer.weight.data.copy_(W)
    h = GPTQ(layer, group_size=128, sym=True, rel_damp=0.01, block_size=128, quantization_order=order)
    h.update(X[:100].to(dev))
    h.update(X[100:].to(dev))
    h.symmetrize_hessian()
    _check_H(h.H.cpu(), 1e-5)
    q, s, z = h.quantize(4)
    assert np.array_equal(s.cpu().view(torch.int16).numpy(), G[f"scale_bits_{tag}"])
    match = (q.cpu().numpy() == G[f"qweight_{tag}"]).mean()
    assert match >= 0.999, match
    packed = pack_weight({"qweight": q, "scale": s, "zero": z}, 4, True, 128)["weight_packed"]
    want = O.pack_to_int32(q.cpu().to(torch.int8) - 8, 4)  # bit-exact given the same codes
    assert torch.equal(packed.cpu(), want)
    assert torch.equal(h.packed_words().cpu(), want)
    if match == 1.0:
        assert np.array_equal(packed.cpu().numpy(), G[f"packed_{tag}"])
