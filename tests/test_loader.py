"""Checkpoint -> layer: compressed-tensors `int-quantized` expert tensors (format of
docs/source/tutorials/multi_xpu_DeepSeek-V3.2-Exp-w8a8.md:50-95) through the method
selection of compressed_tensors_moe.py:43-108 and the expert mapping of
models/deepseek_v2.py:1296-1384. Host logic: runs without a GPU."""
import json

import pytest
import torch

import vllm_kunlun_amd  # noqa: F401
from vllm_kunlun_amd.ops.fused_moe.layer import FusedMoE, KunlunUnquantizedFusedMoEMethod
from vllm_kunlun_amd.quantization.compressed_tensors.compressed_tensors import CompressedTensorsConfig
from vllm_kunlun_amd.quantization.compressed_tensors.compressed_tensors_moe import (
    KunlunCompressedTensorsMoEMethod, KunlunCompressedTensorsW8A8Fp8MoEMethod,
    KunlunCompressedTensorsW8A8Int8MoEMethod)

QUANT_CONFIG = json.loads("""{
  "config_groups": {"group_0": {"format": "int-quantized",
    "input_activations": {"dynamic": true, "group_size": null, "num_bits": 8, "strategy": "token",
                          "symmetric": true, "type": "int"},
    "output_activations": null, "targets": ["Linear"],
    "weights": {"dynamic": false, "group_size": null, "num_bits": 8, "observer": "minmax",
                "strategy": "channel", "symmetric": true, "type": "int"}}},
  "format": "int-quantized", "ignore": ["lm_head"], "quant_method": "compressed-tensors",
  "quantization_status": "compressed", "version": "0.12.2"}""")


def _checkpoint(E, H, I, prefix="model.layers.3.mlp."):
    g = torch.Generator().manual_seed(7)
    t = {}
    for e in range(E):
        for proj, (n, k) in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I))):
            t[f"{prefix}experts.{e}.{proj}.weight"] = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
            t[f"{prefix}experts.{e}.{proj}.weight_scale"] = torch.rand(n, 1, generator=g) * 0.01 + 1e-4
    t[f"{prefix}gate.weight"] = torch.randn(E, H, generator=g).bfloat16()           # not an expert tensor
    t[f"{prefix}shared_experts.gate_proj.weight"] = torch.zeros(I, H, dtype=torch.int8)
    return t


def test_expert_params_mapping_has_the_upstream_shape():
    m = FusedMoE.make_expert_params_mapping("gate_proj", "down_proj", "up_proj", num_experts=9)
    assert len(m) == 27
    assert ("experts.w13_", "experts.7.up_proj.", 7, "w3") in m
    assert ("experts.w13_", "experts.0.gate_proj.", 0, "w1") in m
    assert ("experts.w2_", "experts.8.down_proj.", 8, "w2") in m
    # the way the model loop uses it (models/deepseek_v2.py:1347-1356)
    name = "model.layers.3.mlp.experts.7.up_proj.weight_scale"
    param_name, weight_name, e, shard = next(x for x in m if x[1] in name)
    assert name.replace(weight_name, param_name) == "model.layers.3.mlp.experts.w13_weight_scale"
    with pytest.raises(NotImplementedError):
        FusedMoE.make_expert_params_mapping("gate_proj", "down_proj", "up_proj", 4, num_redundant_experts=1)


def test_method_selection_from_a_checkpoint_config():
    cfg = CompressedTensorsConfig.from_config(QUANT_CONFIG)
    stub = FusedMoE(num_experts=2, top_k=1, hidden_size=64, intermediate_size=32)
    m = KunlunCompressedTensorsMoEMethod.get_moe_method(cfg, stub, "model.layers.3.mlp.experts")
    assert isinstance(m, KunlunCompressedTensorsW8A8Int8MoEMethod)
    cfg.ignore.append(r"re:.*layers\.0\..*")
    m0 = KunlunCompressedTensorsMoEMethod.get_moe_method(cfg, stub, "model.layers.0.mlp.experts")
    assert isinstance(m0, KunlunUnquantizedFusedMoEMethod)
    fp8 = json.loads(json.dumps(QUANT_CONFIG))
    grp = fp8["config_groups"]["group_0"]
    grp["weights"].update(type="float", strategy="block", block_structure=[128, 128])
    grp["input_activations"].update(type="float", strategy="group", group_size=128)
    m8 = KunlunCompressedTensorsMoEMethod.get_moe_method(CompressedTensorsConfig.from_config(fp8), stub, "x.experts")
    assert isinstance(m8, KunlunCompressedTensorsW8A8Fp8MoEMethod)
    w4 = json.loads(json.dumps(QUANT_CONFIG))
    w4["config_groups"]["group_0"]["input_activations"] = None
    w4["config_groups"]["group_0"]["weights"].update(num_bits=4, strategy="group", group_size=128)
    with pytest.raises(ValueError):   # 4-bit weight-only needs the pack-quantized format (reference :76-93)
        KunlunCompressedTensorsMoEMethod.get_moe_method(CompressedTensorsConfig.from_config(w4), stub, "x.experts")
    w4["config_groups"]["group_0"]["format"] = "pack-quantized"
    m4 = KunlunCompressedTensorsMoEMethod.get_moe_method(CompressedTensorsConfig.from_config(w4), stub, "x.experts")
    assert type(m4).__name__ == "KunlunCompressedTensorsWNA16MoEMethod" and m4.group_size == 128
    with pytest.raises(ValueError):
        CompressedTensorsConfig.from_config({"quant_method": "gptq"})


def test_safetensors_checkpoint_loads_into_the_stacked_parameters(tmp_path):
    from safetensors import safe_open
    from safetensors.torch import save_file
    E, H, I = 5, 64, 32
    ckpt = _checkpoint(E, H, I)
    save_file(ckpt, str(tmp_path / "model-00001-of-00001.safetensors"))
    cfg = CompressedTensorsConfig.from_config(QUANT_CONFIG)
    stub = FusedMoE(num_experts=E, top_k=2, hidden_size=H, intermediate_size=I)
    method = KunlunCompressedTensorsMoEMethod.get_moe_method(cfg, stub, "model.layers.3.mlp.experts")
    layer = FusedMoE(num_experts=E, top_k=2, hidden_size=H, intermediate_size=I, quant_method=method)

    def tensors():
        with safe_open(str(tmp_path / "model-00001-of-00001.safetensors"), framework="pt") as f:
            for name in f.keys():
                yield name, f.get_tensor(name)

    loaded = layer.load_weights(tensors())
    assert len(loaded) == 6 * E and all(".experts." in n for n in loaded)
    p = "model.layers.3.mlp."
    for e in range(E):
        assert torch.equal(layer.w13_weight[e, :I], ckpt[f"{p}experts.{e}.gate_proj.weight"])
        assert torch.equal(layer.w13_weight[e, I:], ckpt[f"{p}experts.{e}.up_proj.weight"])
        assert torch.equal(layer.w2_weight[e], ckpt[f"{p}experts.{e}.down_proj.weight"])
        assert torch.equal(layer.w13_weight_scale[e, I:], ckpt[f"{p}experts.{e}.up_proj.weight_scale"])
        assert torch.equal(layer.w2_weight_scale[e], ckpt[f"{p}experts.{e}.down_proj.weight_scale"])
    before = layer.w2_weight_scale.clone()
    method.process_weights_after_loading(layer)       # scale -> absmax (reference :116-120); no tiling on the host
    assert torch.equal(layer.w2_weight_scale, before * 127.0)


def test_weight_loader_rejects_what_does_not_fit():
    layer = FusedMoE(num_experts=2, top_k=1, hidden_size=64, intermediate_size=32,
                     quant_method=KunlunCompressedTensorsW8A8Int8MoEMethod())
    with pytest.raises(ValueError):
        layer.weight_loader(layer.w13_weight, torch.zeros(31, 64, dtype=torch.int8), "x", shard_id="w1", expert_id=0)
    with pytest.raises(ValueError):
        layer.weight_loader(layer.w13_weight, torch.zeros(32, 64, dtype=torch.int8), "x", shard_id="w9", expert_id=0)
    assert layer.weight_loader(layer.w13_weight, torch.zeros(32, 64, dtype=torch.int8), "x", shard_id="w1",
                               expert_id=5, return_success=True) is False     # an expert this layer does not hold
    # per-channel scales given as a vector
    layer.weight_loader(layer.w2_weight_scale, torch.full((64,), 0.5), "x", shard_id="w2", expert_id=1)
    assert torch.all(layer.w2_weight_scale[1] == 0.5) and torch.all(layer.w2_weight_scale[0] == 0)


@pytest.mark.gpu
def test_loaded_layer_computes_what_the_directly_built_layer_does():
    E, H, I, M, K = 8, 256, 128, 40, 2
    ckpt = _checkpoint(E, H, I)
    layers = []
    for how in ("loader", "direct"):
        method = KunlunCompressedTensorsW8A8Int8MoEMethod()
        layer = FusedMoE(num_experts=E, top_k=K, hidden_size=H, intermediate_size=I, quant_method=method,
                         device="cuda")
        if how == "loader":
            layer.load_weights(ckpt.items())
        else:
            p = "model.layers.3.mlp."
            for e in range(E):
                layer.w13_weight.data[e].copy_(torch.cat([ckpt[f"{p}experts.{e}.gate_proj.weight"],
                                                          ckpt[f"{p}experts.{e}.up_proj.weight"]]))
                layer.w13_weight_scale.data[e].copy_(torch.cat([ckpt[f"{p}experts.{e}.gate_proj.weight_scale"],
                                                                ckpt[f"{p}experts.{e}.up_proj.weight_scale"]]))
                layer.w2_weight.data[e].copy_(ckpt[f"{p}experts.{e}.down_proj.weight"])
                layer.w2_weight_scale.data[e].copy_(ckpt[f"{p}experts.{e}.down_proj.weight_scale"])
        method.process_weights_after_loading(layer)
        layers.append(layer)
    with pytest.raises(RuntimeError):  # the codes were re-tiled in place: loading now would corrupt them
        layers[0].weight_loader(layers[0].w13_weight, torch.zeros(I, H, dtype=torch.int8), "x", shard_id="w1",
                                expert_id=0)
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(M, H, generator=g, device="cuda").bfloat16()
    logits = torch.randn(M, E, generator=g, device="cuda")
    a, b = layers[0](x, logits), layers[1](x, logits)
    torch.cuda.synchronize()
    assert torch.equal(a, b) and bool(a.float().abs().sum() > 0)
