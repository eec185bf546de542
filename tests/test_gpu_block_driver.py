"""The per-block driver (hooks -> Hessians -> quantize -> files) on a toy MoE block, every linear checked against
the CPU oracle fed with the inputs that linear actually saw."""
import os

import pytest
import torch
import torch.nn as nn

from moe_quant_amd import block_driver, quant_utils
from oracle import gptq_oracle as O

pytestmark = pytest.mark.gpu

HID, INTER, NEXP = 256, 128, 4


class Expert(nn.Module):
    def __init__(self):
        super().__init__()
        self.gate_proj = nn.Linear(HID, INTER, bias=False)
        self.up_proj = nn.Linear(HID, INTER, bias=False)
        self.down_proj = nn.Linear(INTER, HID, bias=False)

    def forward(self, x):
        return self.down_proj(torch.nn.functional.silu(self.gate_proj(x)) * self.up_proj(x))


class Mlp(nn.Module):
    def __init__(self):
        super().__init__()
        self.experts = nn.ModuleList([Expert() for _ in range(NEXP)])
        self.shared_experts = Expert()
        self.register_buffer("router", torch.randn(HID, NEXP))

    def forward(self, x):
        top = (x.float() @ self.router.float()).topk(2, dim=-1).indices
        out = self.shared_experts(x)
        for e, ex in enumerate(self.experts):
            rows = (top == e).any(-1).nonzero().flatten()
            if rows.numel():
                out = out.index_add(0, rows, ex(x[rows]))
        return out


class Block(nn.Module):
    def __init__(self):
        super().__init__()
        self.self_attn = nn.Module()
        self.self_attn.o_proj = nn.Linear(HID, HID, bias=False)
        self.mlp = Mlp()

    def forward(self, x):
        h = x + self.self_attn.o_proj(x)
        return h + self.mlp(h)


class Toy(nn.Module):
    def __init__(self):
        super().__init__()
        self.model = nn.Module()
        self.model.layers = nn.ModuleList([Block() for _ in range(4)])


@pytest.mark.parametrize("tie,only_experts", [(True, False), (False, True)])
def test_block_driver_against_oracle(dev, tmp_path, tie, only_experts):
    torch.manual_seed(0)
    toy = Toy()
    for p in toy.parameters():
        p.data.mul_(0.5)
    toy = toy.to(dev).to(torch.bfloat16)
    block_idx = 3
    prefix = f"model.layers.{block_idx}."
    block = toy.model.layers[block_idx]
    g = torch.Generator().manual_seed(1)
    seqs = [(torch.randn(600, HID, generator=g)).to(torch.bfloat16).to(dev) for _ in range(3)]

    # what every linear sees, and the original weights
    seen, originals, hooks = {}, {}, []
    for name, layer in block_driver.select_layers(toy, prefix, ".*", block_driver.LINEAR_LAYERS).items():
        seen[name] = []
        originals[name] = layer.weight.detach().cpu().clone()
        hooks.append(layer.register_forward_hook(lambda m, inp, out, n=name: seen[n].append(inp[0].detach().cpu())))
    for x in seqs:
        block(x)
    for h in hooks:
        h.remove()

    save_dir = str(tmp_path / "q")
    rep = block_driver.quantize_block(toy, prefix, lambda: [block(x) for x in seqs], bits=4, group_size=128,
                                      tie_gptq_handles=tie, quantize_only_experts=only_experts, save_dir=save_dir,
                                      log_error=True, streams=3)
    block_driver.save_metadata(save_dir, 4, 128, only_experts)
    expect = [n for n in seen if (not only_experts) or ".mlp.experts." in n]
    assert sorted(rep.layers) == sorted(expect)
    assert rep.shared == {"zero_samples": 0, "nan_hessian": 0, "non_invertible": 0} == rep.experts
    for name in expect:
        W = originals[name]
        src = name.replace("up_proj", "gate_proj") if (tie and name.endswith("up_proj")) else name
        Href, n = None, 0
        for x in seen[src]:
            if x.shape[0]:
                Href, n = O.hessian_update(Href, n, x)
        assert rep.tokens_collected[name] == n
        ref = O.quantize_linear(W, Href)
        blob = torch.load(os.path.join(save_dir, name, "quantized_weight.pt"), weights_only=True)
        assert set(blob) == {"qweight", "scale", "zero"}
        q, s, z = blob["qweight"].cpu(), blob["scale"].cpu(), blob["zero"].cpu()
        assert q.dtype == torch.uint8 and s.dtype == torch.bfloat16
        assert torch.equal(s, ref["scale"]) and torch.equal(z, ref["zero"])
        assert (q == ref["qweight"]).float().mean().item() >= 0.999, name
        layer = dict(toy.named_modules())[name]
        assert torch.equal(layer.weight.data.cpu(), O.dequantize_linear_weight(q, s, z))  # weight replaced (quant.py:328)
        assert 0 < rep.relative_error[name] < 0.1
    for name in seen:
        if name not in expect:  # untouched
            assert torch.equal(dict(toy.named_modules())[name].weight.data.cpu(), originals[name])
    meta = torch.load(os.path.join(save_dir, "metadata.pt"), weights_only=True)
    assert meta == {"bits": 4, "group_size": 128, "quantize_only_experts": only_experts}
    assert block_driver.get_resume_block_idx(save_dir) == block_idx


def test_pack_block_after_driver(dev, tmp_path):
    """quantized_weight.pt files -> packed safetensors shard + index + quantization_config, read back and unpacked."""
    import json

    from safetensors.torch import load_file

    from moe_quant_amd import pack_quantized_model as P

    torch.manual_seed(0)
    toy = Toy().to(dev).to(torch.bfloat16)
    block_idx = 2
    prefix = f"model.layers.{block_idx}."
    block = toy.model.layers[block_idx]
    x = torch.randn(500, HID, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16).to(dev)
    qdir, pdir = str(tmp_path / "q"), str(tmp_path / "p")
    block_driver.quantize_block(toy, prefix, lambda: block(x), quantize_only_experts=True, save_dir=qdir)
    block_driver.save_metadata(qdir, 4, 128, True)
    meta = torch.load(os.path.join(qdir, "metadata.pt"), weights_only=True)
    names = P.quantized_layers_by_block(qdir)
    assert list(names) == [block_idx] and len(names[block_idx]) == 3 * NEXP
    sd = {f"{prefix}{k}": v.detach().cpu() for k, v in block.state_dict().items()}
    sd = P.pack_block_state_dict(sd, qdir, names[block_idx], meta["bits"], True, meta["group_size"])
    index = {}
    shard = P.save_packed_shard(sd, pdir, block_idx + 2, 6, index)
    P.save_safetensors_index(pdir, index)
    back = load_file(os.path.join(pdir, shard))
    wm = json.load(open(os.path.join(pdir, "model.safetensors.index.json")))["weight_map"]
    assert set(wm) == set(back) == set(sd)
    for name in names[block_idx]:
        blob = torch.load(os.path.join(qdir, name, "quantized_weight.pt"), weights_only=True)
        assert f"{name}.weight" not in back
        words, shape = back[f"{name}.weight_packed"], back[f"{name}.weight_shape"]
        assert words.dtype == torch.int32 and shape.tolist() == list(blob["qweight"].shape)
        assert torch.equal(O.unpack_from_int32(words, 4, shape.tolist()), blob["qweight"].cpu().to(torch.int8) - 8)
        assert torch.equal(back[f"{name}.weight_scale"], blob["scale"].cpu())
    assert f"{prefix}self_attn.o_proj.weight" in back  # untouched tensors travel along
    cfg = P.prepare_quantization_config(meta["bits"], meta["group_size"], meta["quantize_only_experts"])
    w = cfg["config_groups"]["group_0"]["weights"]
    assert cfg["format"] == "pack-quantized" and w["num_bits"] == 4 and w["group_size"] == 128 and w["symmetric"]
    assert "re:.*shared_experts.*" in cfg["ignore"] and cfg["ignore"][0] == "lm_head"
