"""The allocation-free variant of the damping step (mq_hessian_damp_noalloc: scratch memory inside the library)
against mq_hessian_damp with a caller workspace: bit-identical H, flags and behaviour, on two calls in a row, the
second smaller than the first (the shared scratch array keeps the first call's contents)."""
import pytest
import torch

from moe_quant_amd import _lib, ops, synth

pytestmark = pytest.mark.gpu


def _problem(dev, R, C, seed, dtype=torch.bfloat16):
    X = synth.activations_outlier(C + 64, C, seed)
    X[:, 5] = 0  # a dead input channel
    H = torch.zeros(C, C, device=dev)
    ops.hessian_syrk_(H, X.to(dev), 0.0, 2.0 / X.shape[0])
    W = synth.weight(R, C, seed + 1).float().to(dtype)
    W[:, 9] = 0  # an all-zero weight column
    W[:, C - 1] = 0
    return H, W.to(dev)


def _both(dev, R, C, seed, dtype=torch.bfloat16):
    print(f"no-alloc damp R={R} C={C} seed={seed} {dtype}", flush=True)
    H, W = _problem(dev, R, C, seed, dtype)
    Ha, Hb = H.clone(), H.clone()
    pa, fa = ops.hessian_prestep_(Ha, False)
    pb, fb = ops.hessian_prestep_(Hb, False)
    ops.hessian_damp_(Ha, W, pa, 0.01, fa)
    ops.hessian_damp_noalloc_(Hb, W, pb, 0.01, fb)
    torch.cuda.synchronize()
    assert torch.equal(Ha, Hb) and torch.equal(fa, fb) and torch.equal(pa, pb)
    assert int(fb[2].item()) == 3 and int(fb[1].item()) == 1  # channels 5 (pruned), 9 and C-1 (zero weights)
    assert not torch.equal(Hb, H)
    d = Hb.diagonal()
    assert d[5].item() == d[9].item() and Hb[9, :9].abs().max().item() == 0.0


def test_noalloc_damp_equals_workspace_damp_twice_second_smaller(dev):
    _both(dev, 512, 1536, 1)
    _both(dev, 96, 384, 2)  # smaller: the scratch array still holds the masks of the 1536-channel call
    _both(dev, 200, 1000, 3, torch.float32)  # unaligned width, fp32 weights: the scalar scan path


def test_noalloc_damp_allocates_nothing(dev):
    """What the entry point is for: after the first call on a device (which looks up the scratch array's address),
    a call neither takes memory from torch's allocator nor from the device behind its back."""
    H, W = _problem(dev, 128, 768, 4)
    pruned, flags = ops.hessian_prestep_(H, False)
    ops.hessian_damp_noalloc_(H, W, pruned, 0.01, flags)  # first call: the one-time symbol lookup
    torch.cuda.synchronize()
    before = (torch.cuda.memory_allocated(dev), torch.cuda.memory_reserved(dev), torch.cuda.mem_get_info(dev)[0])
    for _ in range(3):
        ops.hessian_damp_noalloc_(H, W, pruned, 0.01, flags)
    torch.cuda.synchronize()
    after = (torch.cuda.memory_allocated(dev), torch.cuda.memory_reserved(dev), torch.cuda.mem_get_info(dev)[0])
    assert before == after, (before, after)


def test_noalloc_damp_refuses_what_does_not_fit(dev):
    lib = _lib.load()
    flags = torch.zeros(4, dtype=torch.int32, device=dev)
    H = torch.zeros(8, 8, device=dev)
    W = torch.zeros(8, 8, device=dev)
    rc = lib.mq_hessian_damp_noalloc(H.data_ptr(), 40000, 40000, W.data_ptr(), 0, 40000, 8, None, 0.01, flags.data_ptr(), None)
    assert rc == _lib.MQ_ERR_TOO_LARGE
    torch.cuda.synchronize()
    assert torch.equal(flags.cpu(), torch.zeros(4, dtype=torch.int32))  # nothing ran
