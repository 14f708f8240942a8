"""The dense W8A8 linear kernel class (reference: quantization/kernels/scale_mm.py:30-90): what
process_weights_after_loading leaves on the layer (CPU), and apply_weights against the oracle's
quantise -> int8 GEMM -> rescale on the GPU, bit for bit."""
import os
import sys
from types import SimpleNamespace

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "vllm-kunlun_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

from conftest import bits, from_bits  # noqa: E402
from oracle import c_oracle as co  # noqa: E402
from oracle import torch_moe as tm  # noqa: E402


def _layer(n, k, device, seed):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(n, k, generator=g) * 0.05
    wq, scale = tm.quantize_weight_per_channel(w)  # int8 [n,k], scale [n,1] as a checkpoint stores it
    layer = SimpleNamespace(weight=torch.nn.Parameter(wq.to(device), requires_grad=False),
                            weight_scale=torch.nn.Parameter(scale.clone().to(device), requires_grad=False),
                            input_scale=None)
    return layer, wq, (scale * 127.0).reshape(n)  # the absmax the kernels take


def test_process_weights_after_loading_on_the_host():
    from vllm_kunlun_amd.quantization.kernels.scale_mm import (Int8ScaledMMLinearLayerConfig,
                                                               KunlunScaledMMLinearKernel)
    layer, wq, w_max = _layer(48, 96, "cpu", 0)
    scale_before = layer.weight_scale.data.clone()
    kern = KunlunScaledMMLinearKernel(Int8ScaledMMLinearLayerConfig())
    kern.process_weights_after_loading(layer)
    # scale -> absmax: x 127 (scale_mm.py:43-50); one f32 per output channel
    assert torch.equal(layer.weight_scale.data, scale_before * 127.0)
    assert layer.weight_scale.shape == (48, 1) and layer.weight_scale.dtype == torch.float32
    # the base class leaves the weight as the [k, n] transpose view of its [n, k] storage
    assert layer.weight.shape == (96, 48)
    assert torch.equal(layer.weight.data.t(), wq)  # not a HIP tensor: stays row-major
    assert layer.input_scale is None and layer.input_zero_point is None and layer.azp_adj is None
    # a per-tensor scale becomes one per channel
    layer2, _, _ = _layer(32, 64, "cpu", 1)
    layer2.weight_scale = torch.nn.Parameter(torch.tensor([0.25]), requires_grad=False)
    kern.process_weights_after_loading(layer2)
    assert torch.equal(layer2.weight_scale.data, torch.full((32, 1), 0.25 * 127.0))
    # schemes outside the path are refused by name
    ok, why = KunlunScaledMMLinearKernel.can_implement(Int8ScaledMMLinearLayerConfig(is_static_input_scheme=True))
    assert ok and why is None
    ok, why = KunlunScaledMMLinearKernel.can_implement(Int8ScaledMMLinearLayerConfig(input_symmetric=False))
    assert ok and why is None
    # asymmetric activations: the sums of the weight codes per output channel, times the zero point when it is static
    layer3, wq3, _ = _layer(32, 64, "cpu", 3)
    KunlunScaledMMLinearKernel(Int8ScaledMMLinearLayerConfig(input_symmetric=False)).process_weights_after_loading(layer3)
    assert layer3.azp_adj.dtype == torch.int32 and torch.equal(layer3.azp_adj.data, wq3.int().sum(1).reshape(1, 32))
    layer4, wq4, _ = _layer(32, 64, "cpu", 4)
    layer4.input_scale = torch.nn.Parameter(torch.tensor([0.02]), requires_grad=False)
    layer4.input_zero_point = torch.nn.Parameter(torch.tensor([-7], dtype=torch.int32), requires_grad=False)
    KunlunScaledMMLinearKernel(Int8ScaledMMLinearLayerConfig(is_static_input_scheme=True, input_symmetric=False)
                               ).process_weights_after_loading(layer4)
    assert torch.equal(layer4.azp_adj.data, -7 * wq4.int().sum(1).reshape(1, 32)) and layer4.input_scale is not None
    # a fused layer's per-partition static input scales collapse to one: the largest (symmetric) ...
    layer5, _, _ = _layer(32, 64, "cpu", 5)
    layer5.input_scale = torch.nn.Parameter(torch.tensor([0.02, 0.05, 0.03]), requires_grad=False)
    KunlunScaledMMLinearKernel(Int8ScaledMMLinearLayerConfig(is_static_input_scheme=True)).process_weights_after_loading(layer5)
    assert torch.equal(layer5.input_scale.data, torch.tensor([0.05]))
    # ... or the scale and zero point of the range that all partitions cover (asymmetric): partitions
    # [-1.0, 1.55] (scale 0.01, zp -28) and [-0.64, 4.46] (scale 0.02, zp -96) -> [-1.0, 4.46] in 255 steps
    layer6, wq6, _ = _layer(32, 64, "cpu", 6)
    layer6.input_scale = torch.nn.Parameter(torch.tensor([0.01, 0.02]), requires_grad=False)
    layer6.input_zero_point = torch.nn.Parameter(torch.tensor([-28, -96], dtype=torch.int32), requires_grad=False)
    KunlunScaledMMLinearKernel(Int8ScaledMMLinearLayerConfig(is_static_input_scheme=True, input_symmetric=False)
                               ).process_weights_after_loading(layer6)
    want_scale = (0.02 * (127 + 96) - 0.01 * (-128 + 28)) / 255.0
    assert abs(float(layer6.input_scale.data) - want_scale) < 1e-7 and layer6.input_scale.numel() == 1
    want_zp = round(-128 - (0.01 * (-128 + 28)) / want_scale)
    assert int(layer6.input_zero_point.data) == want_zp and layer6.input_zero_point.numel() == 1
    assert torch.equal(layer6.azp_adj.data, want_zp * wq6.int().sum(1).reshape(1, 32))
    with pytest.raises(ValueError):
        bad, _, _ = _layer(16, 64, "cpu", 2)
        bad.weight_scale = torch.nn.Parameter(torch.ones(5), requires_grad=False)
        kern.process_weights_after_loading(bad)


@pytest.mark.gpu
@pytest.mark.parametrize("M,n,k", [(1, 64, 128), (37, 256, 512), (128, 512, 1024), (700, 256, 256),
                                   (5, 48, 80)])  # the last one does not tile: row-major weights
def test_apply_weights_matches_the_oracle(M, n, k):
    from vllm_kunlun_amd import _plan
    from vllm_kunlun_amd.quantization.kernels.scale_mm import KunlunScaledMMLinearKernel
    layer, wq, w_max = _layer(n, k, "cuda", M + n + k)
    kern = KunlunScaledMMLinearKernel()
    kern.process_weights_after_loading(layer)
    assert _plan.is_tiled(layer._kmoe_w_1nk) == (n % 16 == 0 and k % 64 == 0)
    g = torch.Generator().manual_seed(M)
    x = (torch.randn(3, M, k, generator=g) * 1.5).bfloat16()  # leading dimensions are flattened
    out = kern.apply_weights(layer, x.cuda())
    torch.cuda.synchronize()
    assert out.shape == (3, M, n) and out.dtype == torch.bfloat16
    xq, x_max = co.quant_i8_rows(bits(x.reshape(-1, k)))
    lod = np.array([0, 3 * M], dtype=np.int32)
    ref, _ = co.grouped_gemm_i8(xq, x_max, wq.numpy()[None], w_max.numpy()[None], lod)
    assert np.array_equal(bits(out.reshape(-1, n)), ref)
    # with a bias (f32 at the operator, as the reference casts it): a zero bias changes no bit, any other is added in
    # f32 to the rescaled sum before the one rounding (the oracle's epilogue without a zero point, on the maxes)
    out0 = kern.apply_weights(layer, x.cuda(), bias=torch.zeros(n, dtype=torch.bfloat16, device="cuda"))
    bias = torch.randn(n, generator=g).bfloat16()
    out1 = kern.apply_weights(layer, x.cuda(), bias=bias.cuda())
    torch.cuda.synchronize()
    assert torch.equal(out0, out)
    ref1 = co.scaled_mm_azp(xq, wq.numpy(), x_max, w_max.numpy(), None, None, bias.float().numpy())
    assert np.array_equal(bits(out1.reshape(-1, n)), ref1)


@pytest.mark.gpu
@pytest.mark.parametrize("M,n,k,dtype", [(1, 64, 128, torch.bfloat16), (37, 256, 512, torch.float16),
                                         (300, 512, 1024, torch.bfloat16), (5, 48, 80, torch.bfloat16)])
def test_apply_weights_with_a_static_input_scale(M, n, k, dtype):
    """The static symmetric scheme (scale_mm.py:60-66 and 83-90 in the reference: the layer's one input scale
    quantises the tensor, and the GEMM takes scale x 127 as every row's max): codes and output against the
    oracle, bit for bit; values beyond 127 x scale saturate."""
    from vllm_kunlun_amd.quantization.kernels.scale_mm import (Int8ScaledMMLinearLayerConfig,
                                                               KunlunScaledMMLinearKernel)
    layer, wq, w_max = _layer(n, k, "cuda", M + n + k)
    scale = np.float32(0.021)
    layer.input_scale = torch.nn.Parameter(torch.tensor([scale], device="cuda"), requires_grad=False)
    kern = KunlunScaledMMLinearKernel(Int8ScaledMMLinearLayerConfig(is_static_input_scheme=True))
    kern.process_weights_after_loading(layer)
    assert layer.input_scale is not None
    x = (torch.randn(M, k, generator=torch.Generator().manual_seed(M)) * 1.5).to(dtype)  # |x| up to ~6: some saturate
    out = kern.apply_weights(layer, x.cuda())
    torch.cuda.synchronize()
    f16 = dtype == torch.float16
    xq = co.quant_i8_static(bits(x), scale, f16=f16)
    assert (np.abs(xq.astype(np.int32)) == 127).any() or M < 5
    x_max = np.full(M, scale * np.float32(127.0), np.float32)
    ref, _ = co.grouped_gemm_i8(xq, x_max, wq.numpy()[None], w_max.numpy()[None], np.array([0, M], np.int32), f16=f16)
    assert out.dtype == dtype and np.array_equal(bits(out), ref)


@pytest.mark.gpu
@pytest.mark.parametrize("M,n,k,dtype", [(1, 64, 128, torch.bfloat16), (37, 256, 512, torch.float16),
                                         (300, 512, 1024, torch.bfloat16), (5, 48, 80, torch.bfloat16)])
@pytest.mark.parametrize("static", [False, True])
@pytest.mark.parametrize("with_bias", [False, True])
def test_apply_weights_with_asymmetric_activations(M, n, k, dtype, static, with_bias):
    """The asymmetric schemes (scale_mm.py:60-82 in the reference): codes with a zero point per token (dynamic) or
    the layer's own (static), the int8 product and the zero-point correction in the epilogue of
    `_C::cutlass_scaled_mm_azp`: against the oracle's quantisation and its restated epilogue, bit for bit; and
    against the plain float product of x and the dequantised weights within the quantisation error."""
    from vllm_kunlun_amd.quantization.kernels.scale_mm import (Int8ScaledMMLinearLayerConfig,
                                                               KunlunScaledMMLinearKernel)
    layer, wq, w_max = _layer(n, k, "cuda", M + n + k)
    scale, zp = np.float32(0.03), -11
    if static:
        layer.input_scale = torch.nn.Parameter(torch.tensor([scale], device="cuda"), requires_grad=False)
        layer.input_zero_point = torch.nn.Parameter(torch.tensor([zp], dtype=torch.int32, device="cuda"),
                                                    requires_grad=False)
    kern = KunlunScaledMMLinearKernel(Int8ScaledMMLinearLayerConfig(is_static_input_scheme=static, input_symmetric=False))
    kern.process_weights_after_loading(layer)
    g = torch.Generator().manual_seed(M)
    x = (torch.randn(M, k, generator=g) * 1.5 + 0.7).to(dtype)  # not centred: the zero point matters
    bias = torch.randn(n, generator=g) if with_bias else None
    out = kern.apply_weights(layer, x.cuda(), None if bias is None else bias.to(dtype).cuda())
    torch.cuda.synchronize()
    f16 = dtype == torch.float16
    adj = wq.numpy().astype(np.int64).sum(1).astype(np.int32)
    # the reference's per-call expression (w_s / 127.0) as torch evaluates it on the device (a product with the
    # reciprocal there, a division on the host: one unit in the last place apart for some channels)
    scale_b = (layer.weight_scale.data / 127.0).reshape(-1).cpu().numpy()
    assert np.allclose(scale_b, (w_max / 127.0).numpy(), rtol=2e-7, atol=0)
    b32 = None if bias is None else bias.to(dtype).float().numpy()
    if static:
        xq = co.quant_i8_static(bits(x), scale, zp, f16=f16)
        ref = co.scaled_mm_azp(xq, wq.numpy(), np.array([scale], np.float32), scale_b, adj * np.int32(zp), None, b32, f16=f16)
    else:
        xq, xs, xz = co.quant_i8_rows_azp(bits(x), f16=f16)
        ref = co.scaled_mm_azp(xq, wq.numpy(), xs, scale_b, adj, xz, b32, f16=f16)
    assert out.dtype == dtype and out.shape == (M, n) and np.array_equal(bits(out), ref)
    want = x.float() @ (wq.float() * (w_max / 127.0).reshape(n, 1)).T + (0 if bias is None else bias.to(dtype).float())
    assert (out.cpu().float() - want).norm() / want.norm() <= (6e-2 if static else 2e-2)


@pytest.mark.gpu
def test_shared_expert_mlp_through_two_linears():
    """The shared expert as the model code runs it (deepseek_v2.py:280-296 in the reference's tree:
    gate_up_proj, silu_and_mul, down_proj): the same bits as the dense MLP of the oracle."""
    import vllm_kunlun_amd  # noqa: F401
    from vllm_kunlun_amd.quantization.kernels.scale_mm import KunlunScaledMMLinearKernel
    M, H, I = 96, 512, 256
    up, w13q, w13_max = _layer(2 * I, H, "cuda", 11)
    down, w2q, w2_max = _layer(H, I, "cuda", 12)
    kern = KunlunScaledMMLinearKernel()
    kern.process_weights_after_loading(up)
    kern.process_weights_after_loading(down)
    x = (torch.randn(M, H, generator=torch.Generator().manual_seed(13)) * 1.5).bfloat16()
    y = kern.apply_weights(up, x.cuda())
    act = torch.empty(M, I, dtype=torch.bfloat16, device="cuda")
    torch.ops._C.silu_and_mul(act, y)
    out = kern.apply_weights(down, act)
    torch.cuda.synchronize()
    lod = np.array([0, M], dtype=np.int32)
    xq, x_max = co.quant_i8_rows(bits(x))
    y_ref, _ = co.grouped_gemm_i8(xq, x_max, w13q.numpy()[None], w13_max.numpy()[None], lod)
    a_ref = co.silu_and_mul(y_ref)
    aq, a_max = co.quant_i8_rows(a_ref)
    ref, _ = co.grouped_gemm_i8(aq, a_max, w2q.numpy()[None], w2_max.numpy()[None], lod)
    assert np.array_equal(bits(y), y_ref)
    assert np.array_equal(bits(out), ref)
    # and the torch restatement of the reference's two scaled_int8_quant -> matmul steps agrees within bf16 rounding
    t_ref = tm.w8a8_dense(x, w13q, w13_max.reshape(-1, 1), w2q, w2_max.reshape(-1, 1))
    assert (out.cpu().float() - t_ref.float()).norm() / t_ref.float().norm() <= 1e-2


@pytest.mark.gpu
def test_ops_on_weights_that_were_tiled_at_load_time():
    """The operators take weights by tensor: `_C::matmul` gets `layer.weight.t()` as in the reference
    (scale_mm.py:83-90) after process_weights_after_loading re-tiled the storage in place, `_C::moe_fc`
    gets the bf16 layer's w13 after KunlunUnquantizedFusedMoEMethod tiled it. Both must see the tiling
    (it belongs to the memory, not to a tensor object) and give the oracle's result; a view that cannot
    be served is refused instead of being read as row-major."""
    import vllm_kunlun_amd  # noqa: F401
    from conftest import rel_l2
    from vllm_kunlun_amd import _plan
    from vllm_kunlun_amd.ops.fused_moe.layer import FusedMoE
    from vllm_kunlun_amd.quantization.kernels.scale_mm import KunlunScaledMMLinearKernel
    M, n, k = 40, 256, 512
    layer, wq, w_max = _layer(n, k, "cuda", 21)
    kern = KunlunScaledMMLinearKernel()
    kern.process_weights_after_loading(layer)
    assert _plan.is_tiled(layer.weight) and layer.weight.shape == (k, n)
    x = (torch.randn(M, k, generator=torch.Generator().manual_seed(22)) * 1.5).bfloat16()
    x_q, x_s, _, _ = torch.ops._C.scaled_int8_quant(x.cuda(), None, None, True)
    out = torch.ops._C.matmul(x_q, layer.weight.transpose(0, 1), torch.bfloat16, x_pc_max=x_s,
                              w_pc_max=layer.weight_scale)
    torch.cuda.synchronize()
    xq, x_max = co.quant_i8_rows(bits(x))
    ref, _ = co.grouped_gemm_i8(xq, x_max, wq.numpy()[None], w_max.numpy()[None], np.array([0, M], np.int32))
    assert np.array_equal(bits(out), ref)
    with pytest.raises(ValueError):  # the [k, n] view itself is not something the kernels can read
        torch.ops._C.matmul(x_q[:, :n].contiguous(), layer.weight, torch.bfloat16, x_pc_max=x_s,
                            w_pc_max=layer.weight_scale[:k])

    # bf16 grouped GEMM on a tiled bf16 layer
    E, H, I, rows = 4, 256, 128, 50
    g = torch.Generator().manual_seed(23)
    moe = FusedMoE(num_experts=E, top_k=2, hidden_size=H, intermediate_size=I, device="cuda")
    w13 = (torch.randn(E, 2 * I, H, generator=g) * 0.05).bfloat16()
    moe.w13_weight.data.copy_(w13)
    moe.quant_method.process_weights_after_loading(moe)
    assert _plan.is_tiled(moe.w13_weight)
    a = torch.randn(rows, H, generator=g).bfloat16()
    lod = torch.tensor([0, 20, 20, 37, 50], dtype=torch.int32)
    y = torch.empty(rows, 2 * I, dtype=torch.bfloat16, device="cuda")
    torch.ops._C.moe_fc(a.cuda(), moe.w13_weight, lod.cuda(), torch.empty(0, dtype=torch.int32, device="cuda"), 2, y)
    torch.cuda.synchronize()
    ref = co.grouped_gemm_bf16(bits(a), bits(w13), lod.numpy())
    assert rel_l2(y, from_bits(ref)) <= 1e-2
