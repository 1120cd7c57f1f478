"""Host logic of FP8 checkpoint ingestion (sglang_amd/fp8.py), on the CPU: config parsing and its errors, parameter shapes,
slicing of checkpoint tensors into merged and tensor-parallel layers, and what process_weights_after_loading leaves behind.
Expected values are written out from the checkpoint tensors themselves (concatenations and slices), following what the
reference's loaders produce (python/sglang/srt/layers/linear.py:733-760, :962-985; quantization/fp8.py:244-341)."""
import json

import pytest
import torch

from sglang_amd.fp8 import Fp8Config, Fp8Linear, Fp8LinearMethod, load_safetensors_dir

FP8 = torch.float8_e4m3fn
BLOCK_CFG = {"quant_method": "fp8", "fmt": "e4m3", "activation_scheme": "dynamic", "weight_block_size": [128, 128]}


def _proj(n, k, g, name):
    w = ((torch.rand(n, k, generator=g) - 0.5) * 896).clamp(-448, 448).to(FP8)
    s = torch.rand((n + 127) // 128, (k + 127) // 128, generator=g) * 1e-2 + 1e-4
    return {f"{name}.weight": w, f"{name}.weight_scale_inv": s}


def _bytes(t):
    return t.view(torch.uint8)


def test_config_parsing_and_errors(tmp_path):
    cfg = Fp8Config.from_config(BLOCK_CFG)
    assert cfg.is_checkpoint_fp8_serialized and cfg.weight_block_size == [128, 128] and cfg.activation_scheme == "dynamic"
    assert Fp8Config.get_name() == "fp8"
    (tmp_path / "config.json").write_text(json.dumps({"quantization_config": dict(BLOCK_CFG, ignored_layers=["lm_head"])}))
    cfg = Fp8Config.from_checkpoint_dir(str(tmp_path))
    assert cfg.is_layer_skipped("lm_head") and not cfg.is_layer_skipped("model.layers.0.mlp.down_proj")
    with pytest.raises(ValueError, match="Unsupported activation scheme"):
        Fp8Config(True, "sometimes")
    with pytest.raises(ValueError, match="only supports fp8-serialized"):
        Fp8Config(False, "dynamic", weight_block_size=[128, 128])
    with pytest.raises(ValueError, match="must have 2 dimensions"):
        Fp8Config(True, "dynamic", weight_block_size=[128])
    with pytest.raises(ValueError, match="only supports dynamic activation"):
        Fp8Config(True, "static", weight_block_size=[128, 128])
    # a 16-bit checkpoint: the weight parameter keeps the checkpoint's type until process_weights_after_loading, no scales
    layer = Fp8Linear(256, [256], Fp8Config(False, "dynamic"))
    assert layer.weight.dtype == torch.bfloat16 and layer.weight_scale is None and layer.input_scale is None


def test_block_alignment_checks_of_create_weights():
    cfg = Fp8Config.from_config(BLOCK_CFG)
    Fp8Linear(7168, [576], cfg)  # a plain replicated layer may end in a partial block (DeepSeek-V3 kv_a_proj_with_mqa)
    with pytest.raises(ValueError, match="output_partition_size = 576 is not divisible"):
        Fp8Linear(7168, [576, 1536], cfg)  # merged: every projection must be whole blocks
    with pytest.raises(ValueError, match="output_partition_size = 192 is not divisible"):
        Fp8Linear(512, [384], cfg, parallel="column", tp_rank=0, tp_size=2)
    with pytest.raises(ValueError, match="input_size_per_partition = 192 is not divisible"):
        Fp8Linear(384, [256], cfg, parallel="row", tp_rank=1, tp_size=2)


def test_method_registers_the_checkpoint_names_on_the_layer():
    """fp8.py:277-341: `weight`, `weight_scale_inv` / `weight_scale`, `input_scale` are parameters of `layer` itself, each
    with the `weight_loader` the layer handed in; a loader that walks `named_parameters()` finds the checkpoint's keys."""
    cfg = Fp8Config.from_config(BLOCK_CFG)
    layer = torch.nn.Module()
    calls = []

    def loader(param, loaded_weight, loaded_shard_id=None):
        calls.append(loaded_shard_id)
        param.data.copy_(loaded_weight)

    method = Fp8LinearMethod(cfg, tp_size=2)
    method.create_weights(layer, 512, [256, 256], 512, 1024, torch.bfloat16, weight_loader=loader)
    names = dict(layer.named_parameters())
    assert set(names) == {"weight", "weight_scale_inv"} and layer.input_scale is None
    assert tuple(layer.weight.shape) == (512, 512) and layer.weight.dtype == FP8 and tuple(layer.weight_scale_inv.shape) == (4, 4)
    assert (layer.weight.input_dim, layer.weight.output_dim) == (1, 0) and layer.weight_scale_inv.weight_loader is loader
    assert layer.logical_widths == [256, 256] and layer.input_size_per_partition == 512 and layer.output_size_per_partition == 512
    assert layer.orig_dtype == torch.bfloat16
    with pytest.raises(RuntimeError, match="never loaded"):
        method.process_weights_after_loading(layer)
    g = torch.Generator().manual_seed(5)
    ckpt = _proj(512, 512, g, "mlp.gate_up_proj")
    for name, param in layer.named_parameters():
        param.weight_loader(param, ckpt[f"mlp.gate_up_proj.{name}"])
    assert calls == [None, None] and torch.equal(_bytes(layer.weight.data), _bytes(ckpt["mlp.gate_up_proj.weight"]))
    method.process_weights_after_loading(layer)
    # the column-parallel check needs tp_size: the same sizes on one rank are a merged layer only
    with pytest.raises(ValueError, match="output_partition_size = 192 is not divisible"):
        Fp8LinearMethod(cfg, tp_size=2).create_weights(torch.nn.Module(), 512, [192], 512, 384, torch.bfloat16)
    Fp8LinearMethod(cfg, tp_size=1).create_weights(torch.nn.Module(), 512, [192], 512, 192, torch.bfloat16)
    # per-tensor static: scales per merged projection, default loader, channelwise after loading
    static = Fp8LinearMethod(Fp8Config.from_config({"quant_method": "fp8", "activation_scheme": "static"}))
    layer = torch.nn.Module()
    static.create_weights(layer, 128, [64, 32], 128, 96, torch.bfloat16)
    assert set(dict(layer.named_parameters())) == {"weight", "weight_scale", "input_scale"}
    layer.weight.weight_loader(layer.weight, torch.zeros(96, 128).to(FP8))
    layer.weight_scale.weight_loader(layer.weight_scale, torch.tensor([0.5, 0.25]))
    layer.input_scale.weight_loader(layer.input_scale, torch.tensor([2.0, 3.0]))
    static.process_weights_after_loading(layer)
    assert tuple(layer.weight.shape) == (128, 96) and tuple(layer.weight_scale.shape) == (96, 1)
    assert layer.weight_scale[:64].eq(0.5).all() and layer.weight_scale[64:].eq(0.25).all() and float(layer.input_scale) == 3.0


def test_layer_loads_through_named_parameters():
    cfg = Fp8Config.from_config(BLOCK_CFG)
    g = torch.Generator().manual_seed(6)
    ckpt = {**_proj(512, 384, g, "q"), **_proj(256, 384, g, "k"), **_proj(256, 384, g, "v")}
    layer = Fp8Linear(384, [512, 256, 256], cfg, parallel="column", tp_rank=1, tp_size=2, bias=True)
    assert [n for n, _ in layer.named_parameters()] == ["weight", "weight_scale_inv", "bias"]
    for shard, proj in enumerate("qkv"):
        ckpt[f"{proj}.bias"] = torch.randn(ckpt[f"{proj}.weight"].shape[0], generator=g).to(torch.bfloat16)
        for name, param in layer.named_parameters():
            param.weight_loader(param, ckpt[f"{proj}.{name}"], shard)
    want = torch.cat([ckpt["q.weight"][256:], ckpt["k.weight"][128:], ckpt["v.weight"][128:]])
    assert torch.equal(_bytes(layer.weight.data), _bytes(want))
    want_s = torch.cat([ckpt["q.weight_scale_inv"][2:], ckpt["k.weight_scale_inv"][1:], ckpt["v.weight_scale_inv"][1:]])
    assert torch.equal(layer.weight_scale_inv.data, want_s)
    assert torch.equal(layer.bias.data, torch.cat([ckpt["q.bias"][256:], ckpt["k.bias"][128:], ckpt["v.bias"][128:]]))
    with pytest.raises(KeyError, match="does not belong"):
        layer.weight_loader(torch.nn.Parameter(torch.zeros(1)), torch.zeros(1))


def test_merged_projection_from_a_safetensors_checkpoint(tmp_path):
    from safetensors.torch import save_file

    g = torch.Generator().manual_seed(0)
    ckpt = {}
    ckpt.update(_proj(384, 512, g, "mlp.gate_proj"))
    ckpt.update(_proj(384, 512, g, "mlp.up_proj"))
    ckpt.update(_proj(512, 384, g, "mlp.down_proj"))
    save_file(ckpt, str(tmp_path / "model-00001-of-00001.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps({"quantization_config": BLOCK_CFG}))
    cfg = Fp8Config.from_checkpoint_dir(str(tmp_path))
    tensors = load_safetensors_dir(str(tmp_path))
    assert set(tensors) == set(ckpt)

    gate_up = Fp8Linear(512, [384, 384], cfg)
    gate_up.load_from(tensors, ["mlp.gate_proj", "mlp.up_proj"])
    assert torch.equal(_bytes(gate_up.weight.data), _bytes(torch.cat([ckpt["mlp.gate_proj.weight"], ckpt["mlp.up_proj.weight"]])))
    assert torch.equal(gate_up.weight_scale_inv.data,
                       torch.cat([ckpt["mlp.gate_proj.weight_scale_inv"], ckpt["mlp.up_proj.weight_scale_inv"]]))
    with pytest.raises(RuntimeError, match="process_weights_after_loading"):
        gate_up(torch.zeros(1, 512))
    gate_up.process_weights_after_loading()  # block-FP8 on gfx950: tensors stay exactly as loaded
    assert torch.equal(_bytes(gate_up.weight.data), _bytes(torch.cat([ckpt["mlp.gate_proj.weight"], ckpt["mlp.up_proj.weight"]])))

    # the same layer split over two column-parallel ranks: each projection's channels are halved, block rows follow
    for rank in range(2):
        part = Fp8Linear(512, [384, 384], Fp8Config.from_config(dict(BLOCK_CFG, weight_block_size=[64, 128])), parallel="column",
                         tp_rank=rank, tp_size=2)
        assert tuple(part.weight.shape) == (384, 512) and tuple(part.weight_scale_inv.shape) == (6, 4)
    for rank in range(3):
        part = Fp8Linear(512, [384, 384], cfg, parallel="column", tp_rank=rank, tp_size=3)
        part.load_from(tensors, ["mlp.gate_proj", "mlp.up_proj"])
        rows = slice(128 * rank, 128 * rank + 128)
        want_w = torch.cat([ckpt["mlp.gate_proj.weight"][rows], ckpt["mlp.up_proj.weight"][rows]])
        want_s = torch.cat([ckpt["mlp.gate_proj.weight_scale_inv"][rank:rank + 1], ckpt["mlp.up_proj.weight_scale_inv"][rank:rank + 1]])
        assert torch.equal(_bytes(part.weight.data), _bytes(want_w)) and torch.equal(part.weight_scale_inv.data, want_s)

    # row-parallel down projection: input features (and scale block columns) are split
    for rank in range(3):
        part = Fp8Linear(384, [512], cfg, parallel="row", tp_rank=rank, tp_size=3)
        part.load_from(tensors, ["mlp.down_proj"])
        assert torch.equal(_bytes(part.weight.data), _bytes(ckpt["mlp.down_proj.weight"][:, 128 * rank:128 * rank + 128]))
        assert torch.equal(part.weight_scale_inv.data, ckpt["mlp.down_proj.weight_scale_inv"][:, rank:rank + 1])


def test_loader_errors():
    cfg = Fp8Config.from_config(BLOCK_CFG)
    g = torch.Generator().manual_seed(1)
    layer = Fp8Linear(256, [256, 256], cfg)
    t = _proj(256, 256, g, "p")
    with pytest.raises(KeyError):
        layer.load_from(t, ["p", "missing"])
    with pytest.raises(ValueError, match="does not fit"):
        layer.weight_loader("weight", torch.zeros(128, 256).to(FP8), 0)
    with pytest.raises(IndexError):
        layer.weight_loader("weight", t["p.weight"], 2)
    with pytest.raises(KeyError):
        layer.weight_loader("weight_scale", torch.ones(1), 0)
    layer.weight_loader("weight", t["p.weight"], 0)
    layer.weight_loader("weight_scale_inv", t["p.weight_scale_inv"], 0)
    with pytest.raises(RuntimeError, match="never loaded"):  # the second projection's scales are still the marker value
        layer.process_weights_after_loading()
    fused = Fp8Linear(256, [256, 256], cfg, parallel="column", tp_rank=0, tp_size=2)
    with pytest.raises(ValueError, match="without its projection index"):
        fused.weight_loader("weight", torch.zeros(512, 256).to(FP8), None)


def test_per_tensor_checkpoint_becomes_per_channel():
    """fp8.py:384-394, :452-460: N scales for N merged projections -> one scale per output channel; the weight is kept as
    its transposed view; a static input scale is the maximum over the projections."""
    cfg = Fp8Config.from_config({"quant_method": "fp8", "activation_scheme": "static"})
    g = torch.Generator().manual_seed(2)
    layer = Fp8Linear(128, [64, 32, 32], cfg, bias=True)
    assert tuple(layer.weight_scale.shape) == (3,) and tuple(layer.input_scale.shape) == (3,)
    tensors = {}
    for name, n, ws, xs in (("q", 64, 0.01, 0.5), ("k", 32, 0.02, 0.7), ("v", 32, 0.03, 0.6)):
        tensors[f"{name}.weight"] = ((torch.rand(n, 128, generator=g) - 0.5) * 100).to(FP8)
        tensors[f"{name}.weight_scale"] = torch.tensor(ws)
        tensors[f"{name}.input_scale"] = torch.tensor(xs)
        tensors[f"{name}.bias"] = torch.randn(n, generator=g).to(torch.bfloat16)
    layer.load_from(tensors, ["q", "k", "v"])
    layer.process_weights_after_loading()
    assert tuple(layer.weight.shape) == (128, 128) and layer.weight.stride(0) == 1  # [K, N] column-major view
    want = torch.cat([torch.full((64,), 0.01), torch.full((32,), 0.02), torch.full((32,), 0.03)]).reshape(-1, 1)
    assert torch.equal(layer.weight_scale.data, want)
    assert float(layer.input_scale) == pytest.approx(0.7) and layer.input_scale.numel() == 1
    assert torch.equal(layer.bias.data, torch.cat([tensors["q.bias"], tensors["k.bias"], tensors["v.bias"]]))
