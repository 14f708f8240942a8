"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py).
CPU: the oracle still reproduces them. GPU: the kernels reproduce the integer and routing
fixtures bit for bit through the C ABI without the oracle; the layer fixture, whose outputs passed
through SiLU, within the layer's tolerance (and the oracle with the device's SiLU table bit for bit)."""
import os

import numpy as np
import pytest
import torch

from conftest import bits, from_bits, rel_l2

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return dict(np.load(os.path.join(GOLD, name), allow_pickle=False))


def test_oracle_reproduces_routing_fixture():
    from oracle import c_oracle as co
    g = load("routing.npz")
    w, ids = co.softmax_topk(g["logits"], 4, True)
    assert np.array_equal(ids, g["softmax_ids"]) and np.array_equal(w, g["softmax_w"])
    assert list(ids[0]) == [0, 1, 2, 3]  # the tied logits of row 0 resolve to the lowest ids
    w, ids = co.sigmoid_group_topk_norm(g["logits"], g["bias"], 4, 4, 2, 2.5)
    assert np.array_equal(ids, g["sigmoid_ids"]) and np.array_equal(w, g["sigmoid_w"])


def test_oracle_reproduces_layer_fixture():
    from oracle import c_oracle as co
    g = load("w8a8_tiny_layer.npz")
    out, inter = co.forward_w8a8(g["x"], g["logits"], g["w13"], g["w13_max"], g["w2"], g["w2_max"], int(g["K"]),
                                 shared=(g["ws13"], g["ws13_max"], g["ws2"], g["ws2_max"]),
                                 out_scale=float(g["out_scale"]), intermediates=True)
    assert np.array_equal(out, g["out"])
    for k in ("topk_ids", "moe_index", "lod", "actq", "down"):
        assert np.array_equal(inter[k], g[k]), k


def test_oracle_reproduces_fp8_fixture():
    from oracle import c_oracle as co
    g = load("fp8_group_quant.npz")
    q, s = co.quant_fp8_group128(g["x"])
    assert np.array_equal(q, g["q"]) and np.array_equal(s, g["scale"])
    assert g["q"][0, 1] == 0x7E and g["q"][0, 2] == 0xFE and g["scale"][0, 0] == 1.0


@pytest.mark.gpu
def test_gpu_routing_matches_fixture():
    from vllm_kunlun_amd import _lib as L
    g = load("routing.npz")
    logits = torch.from_numpy(g["logits"]).cuda()
    bias = torch.from_numpy(g["bias"]).cuda()
    w = torch.empty(16, 4, device="cuda")
    ids = torch.empty(16, 4, dtype=torch.int32, device="cuda")
    L.check(L.lib.kmoe_softmax_topk(L.ptr(logits), 16, 32, 4, 1, L.ptr(w), L.ptr(ids), L.stream()))
    torch.cuda.synchronize()
    assert np.array_equal(ids.cpu().numpy(), g["softmax_ids"]) and np.array_equal(w.cpu().numpy(), g["softmax_w"])
    L.check(L.lib.kmoe_sigmoid_group_topk_norm(L.ptr(logits), L.ptr(bias), 16, 32, 4, 4, 2, 2.5, L.ptr(w), L.ptr(ids),
                                               L.stream()))
    torch.cuda.synchronize()
    assert np.array_equal(ids.cpu().numpy(), g["sigmoid_ids"]) and np.array_equal(w.cpu().numpy(), g["sigmoid_w"])


@pytest.mark.gpu
@pytest.mark.parametrize("pad", [False, True], ids=["checkpoint-shapes", "padded-and-tiled"])
def test_gpu_layer_matches_fixture(pad):
    from vllm_kunlun_amd.ops.fused_moe.layer import FusedMoE
    from vllm_kunlun_amd.quantization.compressed_tensors.compressed_tensors_moe import (
        KunlunCompressedTensorsW8A8Int8MoEMethod)
    g = load("w8a8_tiny_layer.npz")
    E, two_i, H = g["w13"].shape
    K = int(g["K"])
    method = KunlunCompressedTensorsW8A8Int8MoEMethod()
    method.pad_intermediate = pad  # the fixture's intermediate size is no multiple of 64
    layer = FusedMoE(num_experts=E, top_k=K, hidden_size=H, intermediate_size=two_i // 2, quant_method=method,
                     device="cuda")
    layer.w13_weight.data.copy_(torch.from_numpy(g["w13"]))
    layer.w2_weight.data.copy_(torch.from_numpy(g["w2"]))
    layer.w13_weight_scale.data.copy_(torch.from_numpy(g["w13_max"] / 127.0))
    layer.w2_weight_scale.data.copy_(torch.from_numpy(g["w2_max"] / 127.0))
    method.process_weights_after_loading(layer)
    # x/127*127 need not round-trip: install the fixture's maxes exactly
    I = two_i // 2
    Ip = layer.w2_weight.shape[-1]  # padded: gate rows at [0, I), up rows at [Ip, Ip + I)
    assert (Ip != I) == (pad and I % 64 != 0 and H % 64 == 0)
    w13_max = torch.from_numpy(g["w13_max"]).reshape(E, two_i, -1)
    layer.w13_weight_scale.data[:, :I].copy_(w13_max[:, :I])
    layer.w13_weight_scale.data[:, Ip:Ip + I].copy_(w13_max[:, I:])
    layer.w2_weight_scale.data.copy_(torch.from_numpy(g["w2_max"]).reshape(layer.w2_weight_scale.shape))
    shared = tuple(torch.from_numpy(g[k]).cuda() for k in ("ws13", "ws13_max", "ws2", "ws2_max"))
    out = method.apply_monolithic(layer, from_bits(g["x"]).cuda(), torch.from_numpy(g["logits"]).cuda(),
                                  shared_expert=shared, out_scale=float(g["out_scale"]))
    torch.cuda.synchronize()
    # Bit for bit against the oracle on the fixture's inputs (under a GPU test the oracle applies the device's own
    # SiLU table). The fixture's `out` was written by the oracle with its closed-form SiLU: the hardware's exp2 and
    # reciprocal are within an ulp of it, which moves a few outputs by one 16-bit step - held to rel-L2 <= 1e-2
    # (the tolerance of the layer's 16-bit outputs), with all but a few of the values identical.
    from oracle import c_oracle as co
    shared_np = tuple(g[k] for k in ("ws13", "ws13_max", "ws2", "ws2_max"))
    ref = co.forward_w8a8(g["x"], g["logits"], g["w13"], g["w13_max"], g["w2"], g["w2_max"], K, shared=shared_np,
                          out_scale=float(g["out_scale"]))
    assert np.array_equal(bits(out), ref)
    assert rel_l2(out.cpu(), from_bits(g["out"])) <= 1e-2
    assert np.count_nonzero(bits(out) != g["out"]) <= 0.05 * g["out"].size


@pytest.mark.gpu
def test_gpu_fp8_quant_matches_fixture():
    from vllm_kunlun_amd import _lib as L
    g = load("fp8_group_quant.npz")
    x = from_bits(g["x"]).cuda()
    q = torch.empty(3, 128, dtype=torch.uint8, device="cuda")
    s = torch.empty(3, 1, dtype=torch.float32, device="cuda")
    L.check(L.lib.kmoe_quant_fp8_group128(L.ptr(x), 128, 3, 128, L.ptr(q), 128, L.ptr(s), L.stream()))
    torch.cuda.synchronize()
    assert np.array_equal(q.cpu().numpy(), g["q"]) and np.array_equal(s.cpu().numpy(), g["scale"])
