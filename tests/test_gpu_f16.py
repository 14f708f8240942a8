"""float16 activations on the int8 path (the dtype the reference's deployment recipes run,
ci/scripts/server/start_vllm.sh:26): the whole layer through apply_monolithic and the operator surface,
bit for bit against the C oracle in its half mode, in every kernel regime (weight-streaming decode path,
64-row, 128-row and paced tiles, row-major LDS kernels), with the half form of the caller epilogue
(models/deepseek_v2.py:286-292: routed sum unscaled, shared output times 1/routed_scaling_factor)."""
import numpy as np
import pytest
import torch

from conftest import rel_l2

pytestmark = pytest.mark.gpu

from oracle import c_oracle as co  # noqa: E402
from oracle import torch_moe as tm  # noqa: E402


def hbits(t: torch.Tensor) -> np.ndarray:
    assert t.dtype == torch.float16
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def from_hbits(b: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(b).view(np.int16)).view(torch.float16)


CASES = [
    ("stream-decode-shared", "dsv3-decode", dict(M=40, H=512, E=32, K=4, I=128, n_group=4, topk_group=2, I_shared=128)),
    ("stream-decode-softmax", "qwen3-decode", dict(M=33, H=768, E=24, K=6, I=192)),
    ("short-tiles", "qwen3-decode", dict(M=120, H=512, E=16, K=4, I=256)),
    ("tall-tiles-shared", "dsv3-decode", dict(M=700, H=256, E=8, K=2, I=128, n_group=2, topk_group=1, I_shared=128)),
    ("paced-tiles", "dsv3-decode", dict(M=560, H=512, E=16, K=4, I=256, n_group=4, topk_group=2, I_shared=256)),
    ("rowmajor-lds", "dsv3-decode", dict(M=50, H=272, E=8, K=2, I=80, n_group=2, topk_group=1, I_shared=80)),
    ("shared-other-width", "dsv3-decode", dict(M=37, H=640, E=160, K=6, I=192, n_group=8, topk_group=3,
                                               routed_scale=16.0, I_shared=384)),
]


@pytest.mark.parametrize("name,base,over", CASES, ids=[c[0] for c in CASES])
def test_half_layer_matches_the_oracle(name, base, over):
    from vllm_kunlun_amd import synth
    shape = synth.scaled(synth.SHAPES[base], **over)
    sl = synth.make_w8a8_layer(shape, "cuda", seed=7)
    if name == "rowmajor-lds":
        assert sl.layer.w2_weight.shape[-1] != shape.I or True
    x = (sl.x.float() * 1.5).half()
    method = sl.layer.quant_method
    kw = sl.apply_kwargs()
    # the half form of the caller epilogue: the routing weights stay unscaled, the shared output is scaled down
    scale = shape.routed_scale if shape.scoring == "sigmoid" else 1.0
    if "routed_scaling_factor" in kw:
        kw["routed_scaling_factor"] = 1.0
    shared_scale = 1.0 / scale if sl.shared is not None else 1.0
    out = method.apply_monolithic(sl.layer, x, sl.logits, shared_scale=shared_scale, **kw)
    torch.cuda.synchronize()
    assert out.dtype == torch.float16 and bool(torch.isfinite(out.float()).all())
    w13, w13_max, w2, w2_max, shared = sl.host_weights()
    sh = None if shared is None else tuple(t.numpy() for t in shared)
    ref, inter = co.forward_w8a8(hbits(x), sl.logits.cpu().numpy(), w13.numpy(), w13_max.numpy(), w2.numpy(),
                                 w2_max.numpy(), shape.K, shape.scoring, True, shape.n_group, shape.topk_group, 1.0,
                                 None if sl.bias is None else sl.bias.cpu().numpy(), sh, shared_scale=shared_scale,
                                 intermediates=True, f16=True)
    lay, ws = method.last_layout, method.last_workspace
    ids = ws[lay.topk_ids: lay.topk_ids + 4 * shape.P].view(torch.int32).cpu().numpy().reshape(shape.M, shape.K)
    assert np.array_equal(ids, inter["topk_ids"])
    assert np.array_equal(hbits(out), ref), f"{np.count_nonzero(hbits(out) != ref)} of {ref.size} outputs differ"
    # and the torch expert loop, run in float16
    host = lambda t: None if t is None else t.detach().cpu()  # noqa: E731
    routed = tm.w8a8_moe(host(x), host(sl.logits), w13, w13_max, w2, w2_max, shape.K, shape.scoring, True, shape.n_group,
                         shape.topk_group, 1.0, host(sl.bias))
    if shared is not None:
        routed = routed + tm.w8a8_dense(host(x), *shared) * shared_scale
    assert rel_l2(out, routed) <= 1e-2


def test_half_layer_on_8_wave_tiles_gives_the_same_bits():
    """The wide (8-wave) tiles of the int8 tile kernel (tile_variant 19, 18, 22: 128, 192, 256 rows) in their half
    instantiations: the bits of the default choice, which the cases above compare with the oracle."""
    from vllm_kunlun_amd import _lib as L
    from vllm_kunlun_amd import synth
    from vllm_kunlun_amd._plan import make_moe_plan
    shape = synth.scaled(synth.SHAPES["dsv3-decode"], M=1100, H=512, E=16, K=4, I=256, n_group=4, topk_group=2,
                         I_shared=256)
    sl = synth.make_w8a8_layer(shape, "cuda", seed=21)
    lay = sl.layer
    x = (sl.x.float() * 1.5).half()
    outs = []
    for variant in (0, 6, 19, 18, 22, 17):
        out = torch.empty_like(x)
        plan = make_moe_plan(L.KMOE_FMT_INT8, x, sl.logits, out, shape.K, lay.w13_weight, lay.w2_weight,
                             lay.w13_weight_scale, lay.w2_weight_scale, shape.scoring, True, shape.n_group,
                             shape.topk_group, shape.routed_scale, sl.bias, sl.shared, 1.0, tile_variant=variant)
        plan()
        torch.cuda.synchronize()
        outs.append(out)
    assert bool(torch.isfinite(outs[0].float()).all()) and float(outs[0].float().abs().max()) > 0
    assert all(torch.equal(outs[0], o) for o in outs[1:])


def test_half_layer_with_the_router_gemm_inside():
    from vllm_kunlun_amd import synth
    shape = synth.scaled(synth.SHAPES["qwen3-decode"], M=48, H=512, E=64, K=4, I=128)
    sl = synth.make_w8a8_layer(shape, "cuda", seed=8)
    g = torch.Generator(device="cuda").manual_seed(2)
    x = torch.randn(shape.M, shape.H, generator=g, device="cuda").half()
    w_gate = (torch.randn(shape.E, shape.H, generator=g, device="cuda") * shape.H ** -0.5).half()
    logits = torch.ops._C.router_gemm_bf16_fp32(x, w_gate)
    ref, abs_sum = co.router_gemm(hbits(x), hbits(w_gate), f16=True)
    torch.cuda.synchronize()
    assert np.all(np.abs(logits.cpu().numpy() - ref) <= shape.H * 2.0 ** -24 * abs_sum + 1e-30)
    method = sl.layer.quant_method
    inside = method.apply_monolithic(sl.layer, x, None, router_weight=w_gate)
    outside = method.apply_monolithic(sl.layer, x, logits)
    torch.cuda.synchronize()
    # same logits up to the summation order of the split-K planes: the same experts except at near ties
    assert rel_l2(inside, outside) <= 1e-2


def test_half_operator_surface():
    """quant2d, scaled_int8_quant, moe_fc, matmul, silu_and_mul and moe_post with float16 tensors, and the dense
    W8A8 Linear class, against the oracle's half mode."""
    import vllm_kunlun_amd  # noqa: F401
    from types import SimpleNamespace
    from vllm_kunlun_amd.quantization.kernels.scale_mm import KunlunScaledMMLinearKernel
    g = torch.Generator().manual_seed(9)
    R, k, n, E = 37, 256, 128, 3
    x = (torch.randn(R, k, generator=g) * 2).half()
    xq = torch.empty(R, k, dtype=torch.int8, device="cuda")
    mx = torch.empty(R, 1, dtype=torch.float32, device="cuda")
    torch.ops._C.quant2d(x.cuda(), xq, mx)
    q_ref, mx_ref = co.quant_i8_rows(hbits(x), f16=True)
    assert np.array_equal(xq.cpu().numpy(), q_ref) and np.array_equal(mx.cpu().numpy().ravel(), mx_ref)
    xq2, mx2, _, static = torch.ops._C.scaled_int8_quant(x.cuda(), None, None, True)
    assert not static and torch.equal(xq2, xq) and torch.equal(mx2, mx)
    # grouped GEMM with a half output, plain and fused with SiLU-mul
    w = torch.randint(-127, 128, (E, n, k), generator=g, dtype=torch.int8)
    w_max = torch.rand(E, n, 1, generator=g) * 0.05 + 0.01
    lod = torch.tensor([0, 10, 10, R], dtype=torch.int32)
    idx = torch.empty(0, dtype=torch.int32, device="cuda")
    for act, cols in ((None, n), ("SWISH_GLU", n // 2)):
        y = torch.empty(R, n, dtype=torch.float16, device="cuda")
        torch.ops._C.moe_fc(xq, w.cuda(), lod.cuda(), idx, 1, y, act, mx, w_max.cuda())
        y_ref, _ = co.grouped_gemm_i8(q_ref, mx_ref, w.numpy(), w_max.numpy(), lod.numpy(), act=1 if act else 0, f16=True)
        assert np.array_equal(hbits(y[:, :cols] if act else y), y_ref)
    # silu_and_mul and moe_post
    y = torch.randn(R, 2 * n, generator=g).half()
    out = torch.empty(R, n, dtype=torch.float16, device="cuda")
    torch.ops._C.silu_and_mul(out, y.cuda())
    assert np.array_equal(hbits(out), co.silu_and_mul(hbits(y), f16=True))
    M, K, H = 9, 4, 64
    rows = torch.randn(M * K, H, generator=g).half()
    idx2 = torch.randperm(M * K, generator=g).int().view(M, K)
    wts = torch.rand(M, K, generator=g)
    outp = torch.empty(M, H, dtype=torch.float16, device="cuda")
    torch.ops._C.moe_post(rows.cuda(), idx2.cuda(), wts.cuda(), torch.ones(M, K, device="cuda"), outp)
    assert np.array_equal(hbits(outp), co.combine(hbits(rows), idx2.numpy(), wts.numpy(), f16=True))
    # dense Linear: both the weight-streaming path (few rows) and the tile kernel (many)
    wq, sc = tm.quantize_weight_per_channel(torch.randn(256, 512, generator=g) * 0.05)
    lin = SimpleNamespace(weight=torch.nn.Parameter(wq.cuda(), requires_grad=False),
                          weight_scale=torch.nn.Parameter(sc.clone().cuda(), requires_grad=False), input_scale=None)
    kern = KunlunScaledMMLinearKernel()
    kern.process_weights_after_loading(lin)
    for rows_n in (24, 600):
        xx = (torch.randn(rows_n, 512, generator=g) * 1.5).half()
        got = kern.apply_weights(lin, xx.cuda())
        qq, mm = co.quant_i8_rows(hbits(xx), f16=True)
        ref, _ = co.grouped_gemm_i8(qq, mm, wq.numpy()[None], (sc * 127).reshape(1, -1).numpy(),
                                    np.array([0, rows_n], np.int32), f16=True)
        assert got.dtype == torch.float16 and np.array_equal(hbits(got), ref)
    torch.cuda.synchronize()


def test_float16_is_refused_where_it_is_not_served():
    from vllm_kunlun_amd import synth
    from vllm_kunlun_amd.ops._kunlun_ops import KunlunOps
    shape = synth.scaled(synth.SHAPES["tiny-bf16"], M=8)
    sl = synth.make_bf16_layer(shape, "cuda", seed=1)
    with pytest.raises(ValueError):  # unquantized weights must have the activations' dtype
        sl.layer(sl.x.half(), sl.logits)
    w13, w2 = sl.layer.w13_weight.data.half(), sl.layer.w2_weight.data.half()
    bias = torch.zeros(w13.shape[0], w13.shape[1], dtype=torch.float16, device="cuda")
    with pytest.raises(NotImplementedError):  # the expert-bias branch is bf16 only
        KunlunOps.fused_moe(sl.x.half(), w13, w2, sl.logits, 0, shape.K, True, w1_bias=bias)


# ---------------------------------------------------------------- the unquantized path on half tensors
# (UnquantizedFusedMoEMethod under --dtype float16: activations AND weights are half.) MFMA sums in its own
# order, so these are held to a tolerance like the bf16 path (rel-L2 <= 1e-2 is the bar for 16-bit outputs);
# half carries three more mantissa bits than bf16, and the results sit well inside 1e-3.
REL_L2_HALF = 1e-3

HALF_GEMM_CASES = [
    (1, 64, 128, [16]),
    (4, 64, 256, [3, 0, 17, 1]),
    (2, 256, 1024, [130, 129]),
    (3, 96, 320, [5, 140, 7]),
    (8, 128, 64, [4, 4, 0, 9, 33, 1, 0, 2]),
    (20, 1024, 128, [((53 * i) % 300) for i in range(20)]),
    (2, 96, 160, [140, 3]),        # an odd number of 64-byte steps
]


@pytest.mark.parametrize("E,n,k,counts", HALF_GEMM_CASES)
@pytest.mark.parametrize("tiled,variant", [(False, 1), (False, 2), (False, 3), (True, 0), (True, 1), (True, 2),
                                           (True, 5), (True, 6), (True, 11)])
@pytest.mark.parametrize("act", [0, 1])
def test_unquantized_half_gemm(E, n, k, counts, tiled, variant, act):
    from vllm_kunlun_amd import _lib as L
    torch.manual_seed(E * n + k)
    lod = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    rows = int(lod[-1])
    a = torch.randn(rows, k).half()
    w = (torch.randn(E, n, k) * 0.05).half()
    ref = co.grouped_gemm_bf16(hbits(a), hbits(w), lod, act=act, f16=True)
    n_out = n // 2 if act else n
    da, dw, dl = a.cuda(), w.cuda(), torch.from_numpy(lod).cuda()
    y = torch.zeros(rows, n_out, dtype=torch.float16, device="cuda")
    g = L.GemmBf16Args()
    if tiled:
        dt = torch.empty_like(dw)
        L.check(L.lib.kmoe_tile_weights_i8(dw.data_ptr(), dt.data_ptr(), E, n, 2 * k, L.stream()))
        dw = dt
        g.w_layout = L.KMOE_W_TILED
    g.a, g.lda, g.src_div = da.data_ptr(), k, 1
    g.w, g.lod = dw.data_ptr(), dl.data_ptr()
    g.E, g.n, g.k, g.rows = E, n, k, rows
    g.y, g.ldy, g.act, g.variant = y.data_ptr(), n_out, act, variant
    g.act_dtype = L.KMOE_DT_F16
    L.check(L.lib.kmoe_grouped_gemm_bf16(g, L.stream()))
    torch.cuda.synchronize()
    assert rel_l2(y, from_hbits(ref)) <= 3e-4   # only the summation order differs
    e = int(np.argmax(counts))                  # independent torch check of one expert
    r0, r1 = lod[e], lod[e + 1]
    t = a[r0:r1].float() @ w[e].float().T
    if act:
        gate, up = t[:, : n // 2].half().float(), t[:, n // 2:].half().float()
        t = torch.nn.functional.silu(gate) * up
    assert rel_l2(y[r0:r1], t) <= REL_L2_HALF


@pytest.mark.parametrize("M,tiled", [(40, False), (40, True), (600, True), (3000, True)])
@pytest.mark.parametrize("scoring", ["softmax", "sigmoid"])
def test_unquantized_half_layer(M, tiled, scoring):
    """KunlunOps.fused_moe on half tensors against the oracle's unquantized layer in its half mode: the
    row-major kernels, the decode kernels on tiles, 64-row and 128-row tiles."""
    from vllm_kunlun_amd._plan import tile_pair_
    from vllm_kunlun_amd.ops._kunlun_ops import KunlunOps
    g = torch.Generator().manual_seed(M)
    E, K, H, I = 16, 4, 256, 128
    x = torch.randn(M, H, generator=g).half()
    logits = torch.randn(M, E, generator=g)
    w13 = (torch.randn(E, 2 * I, H, generator=g) * 0.06).half()
    w2 = (torch.randn(E, H, I, generator=g) * 0.09).half()
    bias = torch.randn(E, generator=g) * 0.1 if scoring == "sigmoid" else None
    ref = co.forward_bf16(hbits(x), logits.numpy(), hbits(w13), hbits(w2), K, scoring, True, 4 if bias is not None else 1,
                          2 if bias is not None else 1, 1.0, None if bias is None else bias.numpy(), f16=True)
    d13, d2 = w13.cuda(), w2.cuda()
    if tiled:
        assert tile_pair_(d13, d2)
    out = KunlunOps.fused_moe(x.cuda(), d13, d2, logits.cuda(), 0, K, True, scoring_func=scoring,
                              num_expert_group=4 if bias is not None else None,
                              topk_group=2 if bias is not None else None,
                              e_score_correction_bias=None if bias is None else bias.cuda())
    torch.cuda.synchronize()
    assert out.dtype == torch.float16 and bool(torch.isfinite(out.float()).all())
    assert rel_l2(out, from_hbits(ref)) <= REL_L2_HALF


def test_unquantized_half_moe_fc_op():
    import vllm_kunlun_amd  # noqa: F401
    torch.manual_seed(0)
    E, n, k = 4, 128, 256
    counts = [10, 0, 33, 5]
    lod = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)).cuda()
    rows = sum(counts)
    x = torch.randn(rows, k).half().cuda()
    w = (torch.randn(E, n, k) * 0.05).half().cuda()
    y = torch.zeros(rows, 1, n, dtype=torch.float16, device="cuda")
    idx = torch.arange(rows, dtype=torch.int32, device="cuda")
    torch.ops._C.moe_fc(x, w, lod, idx, 1, y, "SWISH_GLU")
    torch.cuda.synchronize()
    ref = co.grouped_gemm_bf16(hbits(x), hbits(w), lod.cpu().numpy(), act=1, f16=True)
    assert rel_l2(y.view(rows, n)[:, : n // 2], from_hbits(ref)) <= 3e-4
    assert torch.all(y.view(rows, n)[:, n // 2:] == 0)
    with pytest.raises(Exception):  # weight of another dtype
        torch.ops._C.moe_fc(x, w.bfloat16(), lod, idx, 1, y, "SWISH_GLU")


# ---------------------------------------------------------------- packed 4-bit weights with half scales
W4_HALF_CASES = [
    (1, 64, 128, [16], 128),
    (4, 64, 256, [3, 0, 17, 1], 32),
    (8, 256, 1024, [4, 4, 0, 9, 33, 1, 0, 2], 64),
    (2, 128, 512, [70, 3], None),
    (16, 1536, 256, [(5 * i) % 11 for i in range(16)], 128),
    (3, 96, 384, [130, 0, 260], 128),
]


@pytest.mark.parametrize("E,n,k,counts,gs", W4_HALF_CASES)
@pytest.mark.parametrize("variant", [0, 1, 2, 4, 8, 64, 96])
@pytest.mark.parametrize("act", [0, 1])
def test_w4_half_dequant_and_gemm(E, n, k, counts, gs, variant, act):
    """kmoe_dequant_w4 in half mode: the oracle's bits (= the reference's float16 expression). The packed-weight
    GEMM in half mode against unpack + the half unquantized GEMM of the oracle: the operands are the same
    bits, only the summation order differs."""
    from vllm_kunlun_amd import _lib as L
    g = torch.Generator().manual_seed(E * n + k + (gs or 0))
    lod = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    rows = int(lod[-1])
    group = gs or k
    packed = torch.randint(0, 256, (E, n, k // 2), generator=g, dtype=torch.uint8)
    scale = (torch.rand(E, n, k // group, generator=g) * 0.02 + 0.002).half()
    a = torch.randn(rows, k, generator=g).half()
    w_bits = co.dequant_w4_bf16(packed.numpy(), hbits(scale), group, f16=True)
    dp, ds = packed.cuda(), scale.cuda()
    w = torch.empty(E, n, k, dtype=torch.float16, device="cuda")
    L.check(L.lib.kmoe_dequant_w4(dp.data_ptr(), ds.data_ptr(), E * n, k, group, w.data_ptr(), L.KMOE_DT_F16, L.stream()))
    torch.cuda.synchronize()
    assert np.array_equal(hbits(w), w_bits)
    ref = co.grouped_gemm_bf16(hbits(a), w_bits, lod, act=act, f16=True)
    n_out = n // 2 if act else n
    dt = torch.empty_like(dp)
    L.check(L.lib.kmoe_tile_weights_i8(dp.data_ptr(), dt.data_ptr(), E, n, k // 2, L.stream()))
    da, dl = a.cuda(), torch.from_numpy(lod).cuda()
    y = torch.zeros(rows, n_out, dtype=torch.float16, device="cuda")
    args = L.GemmW4Args()
    args.a, args.lda, args.src_div = da.data_ptr(), k, 1
    args.w, args.w_scale, args.group_size, args.lod = dt.data_ptr(), ds.data_ptr(), group, dl.data_ptr()
    args.E, args.n, args.k, args.rows = E, n, k, rows
    args.y, args.ldy, args.act, args.variant, args.w_layout = y.data_ptr(), n_out, act, variant, L.KMOE_W_TILED
    args.act_dtype = L.KMOE_DT_F16
    L.check(L.lib.kmoe_grouped_gemm_w4a16(args, L.stream()))
    torch.cuda.synchronize()
    assert rel_l2(y, from_hbits(ref)) <= 3e-4


@pytest.mark.parametrize("native", ["auto", "both", "only", False])
@pytest.mark.parametrize("group_size,M", [(128, 24), (32, 5), (None, 24), (128, 700)])
def test_w4_half_layer(native, group_size, M):
    """The 4-bit method created with params_dtype float16 (the reference's deployment dtype): half scales, half
    activations; on the packed weights (streaming kernel for the small batches, tile kernel for 700 tokens) or, with
    "both" from 160 rows per expert and with False always, on the copy unpacked once; against the oracle's half
    unquantized layer on the weights its half unpacking gives."""
    from types import SimpleNamespace
    from vllm_kunlun_amd.ops.fused_moe.layer import FusedMoE
    from vllm_kunlun_amd.quantization.compressed_tensors.compressed_tensors_moe import (
        KunlunCompressedTensorsWNA16MoEMethod)
    E, H, I, K = 16, 256, 256, 4
    wq = SimpleNamespace(num_bits=4, type="int", symmetric=True, dynamic=False,
                         strategy="group" if group_size else "channel", group_size=group_size)
    method = KunlunCompressedTensorsWNA16MoEMethod(wq, None, SimpleNamespace(experts_per_token=K), native=native)
    layer = FusedMoE(num_experts=E, top_k=K, hidden_size=H, intermediate_size=I, quant_method=method, device="cuda",
                     params_dtype=torch.float16)
    assert layer.w13_weight_scale.dtype == torch.float16
    g = torch.Generator().manual_seed(11)
    with torch.no_grad():
        for name, (n, k) in (("w13", (2 * I, H)), ("w2", (H, I))):
            getattr(layer, f"{name}_weight_packed").data = torch.randint(0, 256, (E, n, k // 2), generator=g,
                                                                         dtype=torch.uint8).cuda()
            getattr(layer, f"{name}_weight_scale").data = (torch.rand(E, n, k // (group_size or k), generator=g)
                                                           * 0.02 + 0.002).half().cuda()
    packed13, scale13 = layer.w13_weight_packed.data.cpu(), layer.w13_weight_scale.data.cpu()
    packed2, scale2 = layer.w2_weight_packed.data.cpu(), layer.w2_weight_scale.data.cpu()
    method.process_weights_after_loading(layer)
    assert hasattr(layer, "w13_weight") == (native in ("both", False))
    if native in ("both", False):
        assert layer.w13_weight.dtype == torch.float16
    gx = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(M, H, generator=gx, device="cuda").half()
    logits = torch.randn(M, E, generator=gx, device="cuda")
    out = layer(x, logits)
    torch.cuda.synchronize()
    assert out.dtype == torch.float16
    w13 = co.dequant_w4_bf16(packed13.numpy(), hbits(scale13), group_size or H, f16=True)
    w2 = co.dequant_w4_bf16(packed2.numpy(), hbits(scale2), group_size or I, f16=True)
    ref = co.forward_bf16(hbits(x), logits.cpu().numpy(), w13, w2, K, f16=True)
    assert rel_l2(out, from_hbits(ref)) <= REL_L2_HALF
    if native:
        with pytest.raises(ValueError):  # activations of the other 16-bit type
            layer(x[:4].bfloat16(), logits[:4])


def test_w4_half_subnormal_products():
    """Scales so small that (code - 8) * scale is a subnormal half: the unpacking kernels keep them (no flush to
    zero), in the load-time kernel and in the registers of the packed-weight GEMM alike."""
    from vllm_kunlun_amd import _lib as L
    g = torch.Generator().manual_seed(2)
    E, n, k, rows = 1, 64, 128, 16
    packed = torch.randint(0, 256, (E, n, k // 2), generator=g, dtype=torch.uint8)
    scale = (torch.rand(E, n, 1, generator=g) * 4e-6 + 1e-6).half()  # below the smallest normal half (6.1e-5)
    w_bits = co.dequant_w4_bf16(packed.numpy(), hbits(scale), k, f16=True)
    assert (np.abs(from_hbits(w_bits).float().numpy()) < 6.0e-5).all() and (w_bits & 0x7fff).any()
    dp, ds = packed.cuda(), scale.cuda()
    w = torch.empty(E, n, k, dtype=torch.float16, device="cuda")
    L.check(L.lib.kmoe_dequant_w4(dp.data_ptr(), ds.data_ptr(), E * n, k, k, w.data_ptr(), L.KMOE_DT_F16, L.stream()))
    torch.cuda.synchronize()
    assert np.array_equal(hbits(w), w_bits)
    a = (torch.randn(rows, k, generator=g) * 64).half()
    lod = np.array([0, rows], np.int32)
    ref = co.grouped_gemm_bf16(hbits(a), w_bits, lod, f16=True)
    dt = torch.empty_like(dp)
    L.check(L.lib.kmoe_tile_weights_i8(dp.data_ptr(), dt.data_ptr(), E, n, k // 2, L.stream()))
    da, dl = a.cuda(), torch.from_numpy(lod).cuda()
    y = torch.zeros(rows, n, dtype=torch.float16, device="cuda")
    args = L.GemmW4Args()
    args.a, args.lda, args.src_div = da.data_ptr(), k, 1
    args.w, args.w_scale, args.group_size, args.lod = dt.data_ptr(), ds.data_ptr(), k, dl.data_ptr()
    args.E, args.n, args.k, args.rows = E, n, k, rows
    args.y, args.ldy, args.act, args.variant, args.w_layout = y.data_ptr(), n, 0, 0, L.KMOE_W_TILED
    args.act_dtype = L.KMOE_DT_F16
    L.check(L.lib.kmoe_grouped_gemm_w4a16(args, L.stream()))
    torch.cuda.synchronize()
    assert float(from_hbits(ref).float().abs().max()) > 0
    assert rel_l2(y, from_hbits(ref)) <= 2e-3


# ---------------------------------------------------------------- the fp8 block-scaled layer on half activations
@pytest.mark.parametrize("M,I_shared", [(8, 0), (40, 128), (40, 256), (700, 128), (700, 0)])
def test_fp8_layer_with_half_activations(M, I_shared):
    """float16 in, float16 out on fp8 block-scaled weights: the quantiser reads half, the GEMMs round their
    results (and gate and up before SiLU-mul) to half: decode sizes on the LDS-staged kernel, beyond on the tile
    kernel, with a shared expert folded into the routed
    launches (same width), run on its own (another width) or absent; against the oracle in half mode within the
    fp8 tolerance, and against the bfloat16 run of the same layer within what the two output types differ by."""
    from vllm_kunlun_amd import synth
    shape = synth.scaled(synth.SHAPES["dsv3-fp8-decode"], M=M, H=512, E=16, K=4, I=128, n_group=4, topk_group=2,
                         I_shared=I_shared)
    sl = synth.make_layer(shape, "cuda", seed=2, dtype=torch.float16)
    out = sl.layer.quant_method.apply_monolithic(sl.layer, sl.x, sl.logits, **sl.apply_kwargs())
    out_bf = sl.layer.quant_method.apply_monolithic(sl.layer, sl.x.bfloat16(), sl.logits, **sl.apply_kwargs())
    torch.cuda.synchronize()
    assert out.dtype == torch.float16 and bool(torch.isfinite(out.float()).all())
    assert rel_l2(out, out_bf) <= 2e-2
    rows = slice(0, M)
    w13, w13_s, w2, w2_s, sh = sl.host_weights()
    u8 = lambda t: t.view(torch.uint8).numpy()  # noqa: E731
    shared = None if sh is None else (u8(sh[0]), sh[1].numpy(), u8(sh[2]), sh[3].numpy())
    ref = co.forward_fp8(hbits(sl.x[rows]), sl.logits[rows].cpu().numpy(), u8(w13), w13_s.numpy(), u8(w2), w2_s.numpy(),
                         shape.K, shape.scoring, True, shape.n_group, shape.topk_group, shape.routed_scale,
                         sl.bias.cpu().numpy(), shared, f16=True)
    assert rel_l2(out[rows], from_hbits(ref)) <= 3e-2
