"""Writes tests/golden/tiny_gptq.npz: inputs and expected outputs of the CPU oracle for one tiny
linear (R=32, C=256, 288 tokens, g=128, block=128), with and without act-order.

The reference has no fixtures of its own; this file freezes the oracle (itself pinned by
tests/test_oracle.py) so that the HIP path and any later change to the oracle are compared with
the same committed numbers.  Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from moe_quant_amd import synth  # noqa: E402
from oracle import gptq_oracle as O  # noqa: E402


def main():
    torch.set_num_threads(1)  # fixed BLAS summation order
    R, C, n = 32, 256, 288
    W = synth.weight(R, C, 9001)
    X = synth.activations_outlier(n, C, 9002)
    H, _ = O.hessian_update(None, 0, X[:100])
    H, _ = O.hessian_update(H, 100, X[100:])
    out = {"W_bf16_bits": W.view(torch.int16).numpy(), "X_bf16_bits": X.view(torch.int16).numpy(),
           # the Hessian is kept as its diagonal, three full rows and its Frobenius norm (a full copy is 256 KB)
           "H_diag": H.diag().numpy(), "H_rows": H[[0, 100, 255]].numpy(), "H_fro": np.float64(H.double().norm().item())}
    for tag, act in (("default", False), ("actorder", True)):
        r = O.quantize_linear(W, H.clone(), act_order=act)
        out[f"perm_{tag}"] = r["perm"].numpy()
        out[f"qweight_{tag}"] = r["qweight"].numpy()
        out[f"scale_bits_{tag}"] = r["scale"].view(torch.int16).numpy()
        packed = O.pack_weight({"qweight": r["qweight"], "scale": r["scale"], "zero": r["zero"]}, 4, True, 128)
        out[f"packed_{tag}"] = packed["weight_packed"].numpy()
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "tiny_gptq.npz"), **out)
    print("wrote tiny_gptq.npz", {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
