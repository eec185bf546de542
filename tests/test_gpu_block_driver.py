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


def test_pack_command_line_on_a_synthetic_checkpoint(dev, tmp_path):
    """The whole pack step through its command line: a two-block sharded checkpoint (one FP8 tensor with its block
    scales, a stale quantization_config, a tokenizer file) + a quantized directory -> packed shards, weight map and
    config.json; everything read back and checked against the inputs."""
    import json

    from safetensors.torch import load_file, save_file

    from moe_quant_amd import pack_quantized_model as P

    g = torch.Generator().manual_seed(5)
    src, qdir, pdir = tmp_path / "src", tmp_path / "q", tmp_path / "packed"
    src.mkdir()
    R, C = 256, 384
    tensors = {"model.embed_tokens.weight": torch.randn(50, 64, generator=g).bfloat16(),
               "lm_head.weight": torch.randn(50, 64, generator=g).bfloat16(),
               "model.norm.weight": torch.ones(64).bfloat16()}
    qnames = []
    for b in range(2):
        pre = f"model.layers.{b}."
        tensors[pre + "input_layernorm.weight"] = torch.ones(64).bfloat16()
        for proj in ("gate_proj", "down_proj"):
            name = f"{pre}mlp.experts.0.{proj}"
            tensors[name + ".weight"] = (torch.randn(R, C, generator=g) * 0.02).bfloat16()
            qnames.append(name)
    # a layer beyond num_hidden_layers (DeepSeek-V3 ships its multi-token-prediction layer that way): not packed
    tensors["model.layers.2.embed_tokens.weight"] = torch.randn(50, 64, generator=g).bfloat16()
    fp8_name = "model.layers.1.self_attn.o_proj"
    w8 = (torch.randn(R, C, generator=g) * 0.5).to(torch.float8_e4m3fn)
    s8 = torch.rand(R // 128, C // 128, generator=g) * 0.1 + 0.01
    tensors[fp8_name + ".weight"] = w8
    tensors[fp8_name + ".weight_scale_inv"] = s8
    keys = sorted(tensors)
    files = {"model-00001-of-00002.safetensors": keys[: len(keys) // 2], "model-00002-of-00002.safetensors": keys[len(keys) // 2:]}
    wm = {}
    for fn, ks in files.items():
        save_file({k: tensors[k].contiguous() for k in ks}, str(src / fn))
        wm.update({k: fn for k in ks})
    json.dump({"metadata": {}, "weight_map": wm}, open(src / "model.safetensors.index.json", "w"))
    json.dump({"hidden_size": 64, "num_hidden_layers": 2, "quantization_config": {"quant_method": "fp8"}},
              open(src / "config.json", "w"))
    (src / "tokenizer.json").write_text("{}")
    blobs = {}
    for name in qnames:
        W = tensors[name + ".weight"]
        s, z, _ = O.quantization_grid(W.float(), 128, 4, torch.bfloat16)
        q = torch.randint(0, 16, (R, C), generator=g, dtype=torch.uint8)
        blobs[name] = {"qweight": q, "scale": s, "zero": z}
        os.makedirs(qdir / name)
        torch.save(blobs[name], qdir / name / "quantized_weight.pt")
    block_driver.save_metadata(str(qdir), 4, 128, True)
    P.main(["--model_name_or_path", str(src), "--quantized_model_path", str(qdir), "--packed_model_path", str(pdir),
            "--dtype", "bfloat16"])
    out_wm = json.load(open(pdir / "model.safetensors.index.json"))["weight_map"]
    shards = sorted(set(out_wm.values()))
    assert shards == [f"model-{i:05}-of-00004.safetensors" for i in range(1, 5)]
    back = {}
    for fn in shards:
        back.update(load_file(str(pdir / fn)))
    assert set(back) == set(out_wm) and not any(k.startswith("model.layers.2.") for k in back)
    assert out_wm["model.embed_tokens.weight"] == shards[0] and out_wm["lm_head.weight"] == shards[3]
    assert out_wm["model.norm.weight"] == shards[3] and out_wm["model.layers.0.input_layernorm.weight"] == shards[1]
    for name in qnames:
        assert name + ".weight" not in back
        words, shape = back[name + ".weight_packed"], back[name + ".weight_shape"]
        assert shape.tolist() == [R, C]
        assert torch.equal(O.unpack_from_int32(words, 4, [R, C]), blobs[name]["qweight"].to(torch.int8) - 8)
        assert torch.equal(back[name + ".weight_scale"], blobs[name]["scale"])
    assert fp8_name + ".weight_scale_inv" not in back
    rows, cols = torch.arange(R) // 128, torch.arange(C) // 128
    want = w8.to(torch.bfloat16) * s8.to(torch.bfloat16)[rows][:, cols]  # src/quant_utils.py:267-284 in bf16
    assert back[fp8_name + ".weight"].dtype == torch.bfloat16 and torch.equal(back[fp8_name + ".weight"], want)
    for k in ("model.embed_tokens.weight", "lm_head.weight", "model.layers.0.input_layernorm.weight"):
        assert torch.equal(back[k], tensors[k])
    cfg = json.load(open(pdir / "config.json"))
    assert cfg["hidden_size"] == 64 and cfg["quantization_config"]["format"] == "pack-quantized"
    assert cfg["quantization_config"]["config_groups"]["group_0"]["weights"]["group_size"] == 128
    assert "re:.*self_attn.*" in cfg["quantization_config"]["ignore"]
    assert (pdir / "tokenizer.json").exists()


def test_mixed_size_linears_on_three_lanes_equal_one_lane(dev):
    """Linears of very different cost on three lanes (the lanes drift apart) while the driver swaps weights and
    drops Hessians behind the queued kernels: codes, scales and the replaced weights must be bit-identical to the
    one-lane run of the same block."""
    sizes = [(128, 1536), (1024, 256), (256, 128), (128, 1024), (640, 384), (128, 2048), (512, 128), (256, 896)]

    class Bag(nn.Module):
        def __init__(self):
            super().__init__()
            self.lin = nn.ModuleList([nn.Linear(c, r, bias=False) for r, c in sizes])

    def run(streams):
        torch.manual_seed(3)
        bag = Bag().to(dev).to(torch.bfloat16)
        g = torch.Generator().manual_seed(4)
        xs = [torch.randn(700, c, generator=g).to(torch.bfloat16).to(dev) for _, c in sizes]

        def fwd():
            for lin, x in zip(bag.lin, xs):
                lin(x)

        import tempfile

        with tempfile.TemporaryDirectory() as d:
            block_driver.quantize_block(bag, "lin.", fwd, bits=4, group_size=128, save_dir=d, streams=streams)
            blobs = {n: torch.load(os.path.join(d, n, "quantized_weight.pt"), weights_only=True) for n in os.listdir(d)}
        return blobs, [lin.weight.data.clone() for lin in bag.lin]

    b1, w1 = run(1)
    for rep in range(3):
        b3, w3 = run(3)
        assert set(b1) == set(b3) and len(b1) == len(sizes)
        for n in b1:
            for k in ("qweight", "scale", "zero"):
                assert torch.equal(b1[n][k], b3[n][k]), (rep, n, k)
        for a, b in zip(w1, w3):
            assert torch.equal(a, b)
