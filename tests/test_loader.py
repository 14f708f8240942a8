"""Checkpoint -> layer: compressed-tensors `int-quantized` expert tensors (format of
docs/source/tutorials/multi_xpu_DeepSeek-V3.2-Exp-w8a8.md:50-95) through the method
selection of compressed_tensors_moe.py:43-108 and the expert mapping of
models/deepseek_v2.py:1296-1384. The host logic runs without a GPU; the `gpu` tests at the end run the
loaded layer against the oracle on the checkpoint's own tensors."""
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


def _oracle_weights(ckpt, E, prefix="model.layers.3.mlp."):
    """The checkpoint's tensors stacked the way the reference's layer holds them, as numpy arrays for the
    oracle: w13 [E,2I,H] (gate rows first), w2 [E,H,I], and the absmax per channel (= 127 x scale, what
    process_weights_after_loading makes of the scales, compressed_tensors_moe.py:116-120)."""
    import numpy as np
    cat = lambda e, suf: torch.cat([ckpt[f"{prefix}experts.{e}.gate_proj.{suf}"],  # noqa: E731
                                    ckpt[f"{prefix}experts.{e}.up_proj.{suf}"]])
    w13 = torch.stack([cat(e, "weight") for e in range(E)]).numpy()
    w2 = torch.stack([ckpt[f"{prefix}experts.{e}.down_proj.weight"] for e in range(E)]).numpy()
    w13_max = (torch.stack([cat(e, "weight_scale") for e in range(E)]) * 127.0).reshape(E, -1).numpy()
    w2_max = (torch.stack([ckpt[f"{prefix}experts.{e}.down_proj.weight_scale"] for e in range(E)]) * 127.0)
    return w13, w13_max.astype(np.float32), w2, w2_max.reshape(E, -1).numpy().astype(np.float32)


@pytest.mark.gpu
@pytest.mark.parametrize("I", [128, 96])  # 96: padded with zero channels at load time so that the weights tile
def test_loaded_layer_matches_the_oracle_on_the_checkpoint_tensors(I):
    """Checkpoint -> load_weights -> process_weights_after_loading -> forward on the GPU, against the C
    oracle fed with the checkpoint's own tensors (never touched by the loader), bit for bit."""
    import numpy as np
    from conftest import bits
    from oracle import c_oracle as co
    E, H, M, K = 8, 256, 40, 2
    ckpt = _checkpoint(E, H, I)
    method = KunlunCompressedTensorsW8A8Int8MoEMethod()
    layer = FusedMoE(num_experts=E, top_k=K, hidden_size=H, intermediate_size=I, quant_method=method, device="cuda")
    loaded = layer.load_weights(ckpt.items())
    assert len(loaded) == 6 * E
    method.process_weights_after_loading(layer)
    with pytest.raises(RuntimeError):  # the codes were re-tiled in place: loading now would corrupt them
        layer.weight_loader(layer.w13_weight, torch.zeros(I, H, dtype=torch.int8), "x", shard_id="w1", expert_id=0)
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(M, H, generator=g, device="cuda").bfloat16()
    logits = torch.randn(M, E, generator=g, device="cuda")
    out = layer(x, logits)
    torch.cuda.synchronize()
    w13, w13_max, w2, w2_max = _oracle_weights(ckpt, E)
    ref = co.forward_w8a8(bits(x), logits.cpu().numpy(), w13, w13_max, w2, w2_max, K, "softmax", True)
    assert np.array_equal(bits(out), ref)


@pytest.mark.gpu
def test_shared_fused_moe_returns_shared_and_routed_parts():
    """SharedFusedMoE (reference use: models/deepseek_v2.py:241-284) returns (shared_output, routed_output):
    the routed part against the oracle's layer without a shared expert, the shared part (a dense W8A8 MLP of
    two KunlunScaledMMLinearKernel linears, as the model builds it) against the oracle's dense MLP, and their
    caller-side sum `routed * scale + shared` (deepseek_v2.py:288-296) against the oracle's layer with the
    shared expert and the factor folded in - all bit for bit."""
    import numpy as np
    from types import SimpleNamespace
    from conftest import bits, from_bits
    from oracle import c_oracle as co
    from oracle import torch_moe as tm
    from vllm_kunlun_amd.ops.fused_moe.layer import SharedFusedMoE
    from vllm_kunlun_amd.quantization.kernels.scale_mm import KunlunScaledMMLinearKernel
    E, H, I, Is, M, K, scale = 16, 256, 128, 192, 24, 4, 2.5
    ckpt = _checkpoint(E, H, I)
    g = torch.Generator().manual_seed(5)
    kern = KunlunScaledMMLinearKernel()

    def linear(n, k):
        wq, sc = tm.quantize_weight_per_channel(torch.randn(n, k, generator=g) * 0.05)
        lin = SimpleNamespace(weight=torch.nn.Parameter(wq.cuda(), requires_grad=False),
                              weight_scale=torch.nn.Parameter(sc.clone().cuda(), requires_grad=False), input_scale=None)
        kern.process_weights_after_loading(lin)
        return lin, wq.numpy(), (sc * 127.0).reshape(n).numpy()

    up, ws13, ws13_max = linear(2 * Is, H)
    down, ws2, ws2_max = linear(H, Is)

    class SharedMLP(torch.nn.Module):
        def forward(self, x):
            y = kern.apply_weights(up, x)
            act = torch.empty(x.shape[0], Is, dtype=x.dtype, device=x.device)
            torch.ops._C.silu_and_mul(act, y)
            return kern.apply_weights(down, act)

    bias = (torch.randn(E, generator=g) * 0.01).cuda()
    method = KunlunCompressedTensorsW8A8Int8MoEMethod()
    layer = SharedFusedMoE(shared_experts=SharedMLP(), num_experts=E, top_k=K, hidden_size=H, intermediate_size=I,
                           use_grouped_topk=True, num_expert_group=4, topk_group=2, scoring_func="sigmoid",
                           e_score_correction_bias=bias, quant_method=method, device="cuda")
    layer.load_weights(ckpt.items())
    method.process_weights_after_loading(layer)
    x = torch.randn(M, H, generator=g).bfloat16().cuda()
    logits = torch.randn(M, E, generator=g).cuda()
    shared_out, routed_out = layer(x, logits)
    torch.cuda.synchronize()
    assert isinstance(shared_out, torch.Tensor) and shared_out.shape == routed_out.shape == (M, H)
    w13, w13_max, w2, w2_max = _oracle_weights(ckpt, E)
    common = (bits(x), logits.cpu().numpy(), w13, w13_max, w2, w2_max, K, "sigmoid", True, 4, 2, 1.0, bias.cpu().numpy())
    assert np.array_equal(bits(routed_out), co.forward_w8a8(*common))
    lod = np.array([0, M], dtype=np.int32)
    xq, x_max = co.quant_i8_rows(bits(x))
    a_ref = co.grouped_gemm_i8(xq, x_max, ws13[None], ws13_max[None], lod, act=1)[0]
    aq, a_max = co.quant_i8_rows(a_ref)
    sh_ref = co.grouped_gemm_i8(aq, a_max, ws2[None], ws2_max[None], lod)[0]
    assert np.array_equal(bits(shared_out), sh_ref)
    # the caller's epilogue in torch, as the model writes it, equals the oracle's folded epilogue
    final = routed_out * scale + shared_out
    ref = co.forward_w8a8(*common, (ws13, ws13_max, ws2, ws2_max), out_scale=scale)
    assert np.array_equal(bits(final), ref)
    # SharedFusedMoE without a shared module returns (None, routed)
    layer.shared_experts = None
    none_out, routed_again = layer(x, logits)
    assert none_out is None and torch.equal(routed_again, routed_out)


def test_config_get_quant_method_dispatches_on_the_kind_of_layer():
    """KunlunCompressedTensorsConfig.get_quant_method: the call vLLM makes for every layer
    (reference: compressed_tensors.py:49-82)."""
    from vllm_kunlun_amd.quantization.compressed_tensors.compressed_tensors import (
        KunlunCompressedTensorsConfig, KunlunCompressedTensorsW8A8Int8LinearMethod, UnquantizedLinearMethod,
        register_with_vllm)
    from vllm_kunlun_amd.quantization.kernels.scale_mm import KunlunScaledMMLinearKernel
    cfg = KunlunCompressedTensorsConfig.from_config(QUANT_CONFIG)
    assert cfg.get_name() == "compressed-tensors"
    moe = FusedMoE(num_experts=2, top_k=1, hidden_size=64, intermediate_size=32)
    m = cfg.get_quant_method(moe, "model.layers.3.mlp.experts")
    assert isinstance(m, KunlunCompressedTensorsW8A8Int8MoEMethod) and m.moe is moe.moe_config

    class LinearBase(torch.nn.Module):           # stands for vLLM's class of that name
        pass

    class ColumnParallelLinear(LinearBase):
        pass

    lin = ColumnParallelLinear()
    lm = cfg.get_quant_method(lin, "model.layers.3.mlp.shared_experts.gate_up_proj")
    assert isinstance(lm, KunlunCompressedTensorsW8A8Int8LinearMethod)
    assert isinstance(lm.kernel, KunlunScaledMMLinearKernel) and lin.scheme["weights"]["num_bits"] == 8
    lm.create_weights(lin, 64, [32, 32])
    assert lin.weight.shape == (64, 64) and lin.weight.dtype == torch.int8 and lin.weight_scale.shape == (64, 1)
    lm.process_weights_after_loading(lin)        # host: scale -> absmax, weight as the [k, n] view
    assert lin.weight.shape == (64, 64) and lin.input_scale is None
    assert isinstance(cfg.get_quant_method(ColumnParallelLinear(), "lm_head"), UnquantizedLinearMethod)  # ignored
    assert isinstance(cfg.get_quant_method(torch.nn.Linear(4, 4), "model.layers.0.mlp.down_proj"),
                      KunlunCompressedTensorsW8A8Int8LinearMethod)

    class Attention(torch.nn.Module):
        pass

    assert cfg.get_quant_method(Attention(), "model.layers.3.self_attn.attn") is None
    assert cfg.get_quant_method(torch.nn.LayerNorm(4), "model.norm") is None
    # a Linear scheme that is not on the path is refused by name, not served wrongly
    static = json.loads(json.dumps(QUANT_CONFIG))
    static["config_groups"]["group_0"]["input_activations"]["dynamic"] = False
    with pytest.raises(NotImplementedError):
        KunlunCompressedTensorsConfig.from_config(static).get_quant_method(lin, "model.layers.1.mlp.up_proj")
    with pytest.raises(ImportError):             # vLLM is not installed here: the hook says so
        register_with_vllm()
