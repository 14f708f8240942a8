"""GPU parity of the whole W8A8 layer through the plugin surface
(FusedMoE -> quant_method.apply_monolithic -> kmoe_moe_forward in libkmoe.so).

Checked against (1) the C oracle, bit for bit, including the intermediates the
north star names (routing ids, sorted token map, second-GEMM int8 inputs), and
(2) the independently written torch oracle — the reference's per-expert torch
loop — within rel-L2 <= 1e-2 on the bf16 output.
"""
import numpy as np
import pytest
import torch

from conftest import bits, from_bits, rel_l2

pytestmark = pytest.mark.gpu

from oracle import c_oracle as co  # noqa: E402
from oracle import torch_moe as tm  # noqa: E402

REL_L2_BF16 = 1e-2  # north-star tolerance for bf16 outputs of the int8 path


def _host(t):
    return None if t is None else t.detach().cpu()


def _oracle_inputs(sl):
    """Host copies of a SynthLayer's tensors in the oracle's formats."""
    w13, w13_max, w2, w2_max, shared = sl.host_weights()
    if shared is not None:
        shared = tuple(t.numpy() for t in shared)
    return dict(x_bits=bits(sl.x), logits=_host(sl.logits).numpy(), w13=w13.numpy(),
                w13_max=w13_max.numpy(), w2=w2.numpy(),
                w2_max=w2_max.numpy(), K=sl.shape.K, scoring=sl.shape.scoring,
                n_group=sl.shape.n_group, topk_group=sl.shape.topk_group, routed_scale=sl.shape.routed_scale,
                bias=None if sl.bias is None else _host(sl.bias).numpy(), shared=shared)


def _view(ws, off, count, dtype):
    nbytes = count * torch.empty(0, dtype=dtype).element_size()
    return ws[off: off + nbytes].view(dtype)


SMALL = [
    # name, base shape, overrides
    ("softmax-small", "qwen3-decode", dict(M=48, H=512, E=16, K=4, I=256)),
    ("softmax-ragged", "qwen3-decode", dict(M=33, H=768, E=24, K=6, I=160)),
    ("softmax-many-rows", "qwen3-decode", dict(M=700, H=256, E=8, K=2, I=128)),
    # 10 rows per expert: the last batch on the weight-streaming path; 12 and 30: on the tile kernel (64-row tiles
    # that are mostly padding); 60: 128-row tiles
    ("softmax-stream-limit", "qwen3-decode", dict(M=40, H=512, E=16, K=4, I=256)),
    ("softmax-short-tiles", "qwen3-decode", dict(M=120, H=512, E=16, K=4, I=256)),
    ("softmax-tall-tiles-few-rows", "qwen3-decode", dict(M=240, H=512, E=16, K=4, I=256)),
    ("shared-same-width-short-tiles", "dsv3-decode", dict(M=100, H=256, E=8, K=2, I=128, n_group=2, topk_group=1,
                                                          I_shared=128)),
    # expert counts and groupings of other model families (reduced widths): 160 experts in 8 groups of 20 with
    # top-3 groups and top-6 experts; 1000 experts with top-16; a shared expert 20480 wide (rows of more than
    # 16384 values in the second quantisation); hidden 16384
    ("sigmoid-160-experts-8-groups", "dsv3-decode", dict(M=37, H=640, E=160, K=6, I=192, n_group=8, topk_group=3,
                                                         routed_scale=16.0, I_shared=384)),
    # intermediate sizes of tensor-parallel shards (192 = 1536 / 8): an odd number of 64-byte steps in the
    # down projection, on the tile kernel, with and without a shared expert folded into the launches
    ("softmax-shard-192-many-rows", "qwen3-decode", dict(M=500, H=512, E=16, K=4, I=192)),
    ("sigmoid-shard-192-shared-many-rows", "dsv3-decode", dict(M=300, H=640, E=16, K=4, I=192, n_group=4,
                                                               topk_group=2, I_shared=192)),
    ("softmax-1000-experts-top16", "qwen3-decode", dict(M=5, H=256, E=1000, K=16, I=64)),
    ("shared-20480-wide", "dsv3-decode", dict(M=6, H=256, E=8, K=2, I=64, n_group=1, topk_group=1, I_shared=20480)),
    ("hidden-16384", "qwen3-decode", dict(M=3, H=16384, E=8, K=2, I=64)),
    ("sigmoid-grouped-shared", "dsv3-decode", dict(M=40, H=512, E=32, K=4, I=128, n_group=4, topk_group=2,
                                                   I_shared=256)),
    ("sigmoid-flat-shared", "kimi-decode", dict(M=16, H=256, E=48, K=8, I=64, I_shared=128)),
    ("single-token", "qwen3-decode", dict(M=1, H=256, E=8, K=2, I=64)),
    ("shared-same-width-stream", "dsv3-decode", dict(M=40, H=512, E=32, K=4, I=128, n_group=4, topk_group=2,
                                                     I_shared=128)),
    ("shared-same-width-tiled-gemm", "dsv3-decode", dict(M=700, H=256, E=8, K=2, I=128, n_group=2, topk_group=1,
                                                         I_shared=128)),
    ("shared-same-width-rowmajor", "dsv3-decode", dict(M=50, H=272, E=8, K=2, I=80, n_group=2, topk_group=1,
                                                       I_shared=80)),
    # routed weights tile, the shared expert's down projection (k = 32 bytes) cannot: one layout per group
    ("tiled-routed-rowmajor-shared", "dsv3-decode", dict(M=2, H=1024, E=130, K=8, I=256, n_group=2, topk_group=2,
                                                         I_shared=32)),
    ("tiled-routed-rowmajor-shared-many", "dsv3-decode", dict(M=600, H=256, E=8, K=2, I=128, n_group=2,
                                                              topk_group=1, I_shared=32)),
    # the weight-streaming path where its gate_up launch cannot sort the pairs itself (more than 4096 pairs; more
    # than 512 tokens) and where its down launch cannot quantise its rows itself (rows of more than 1024 values)
    ("stream-9600-pairs", "qwen3-decode", dict(M=600, H=256, E=1000, K=16, I=64)),
    ("stream-520-tokens", "qwen3-decode", dict(M=520, H=256, E=256, K=4, I=64)),
    ("stream-512-tokens-4096-pairs", "qwen3-decode", dict(M=512, H=256, E=512, K=8, I=64)),
    ("stream-rows-1088-wide", "qwen3-decode", dict(M=20, H=256, E=16, K=4, I=1088)),
    ("stream-rows-1024-wide", "qwen3-decode", dict(M=20, H=256, E=16, K=4, I=1024)),
    # 17 and 33 channel blocks of 128 in the down projection: the last workgroup's waves partly without channels
    ("stream-down-2112-channels", "qwen3-decode", dict(M=24, H=2112, E=8, K=2, I=128)),
]


@pytest.mark.parametrize("name,base,over", SMALL, ids=[c[0] for c in SMALL])
def test_layer_matches_oracles(name, base, over):
    from vllm_kunlun_amd import synth
    shape = synth.scaled(synth.SHAPES[base], **over)
    _check_layer(synth.make_w8a8_layer(shape, "cuda", seed=1))


def _check_layer(sl):
    shape = sl.shape
    method = sl.layer.quant_method
    out_scale = 1.0
    out = method.apply_monolithic(sl.layer, sl.x, sl.logits, out_scale=out_scale, **sl.apply_kwargs())
    torch.cuda.synchronize()

    oi = _oracle_inputs(sl)
    ref_bits, inter = co.forward_w8a8(**oi, out_scale=out_scale, intermediates=True)

    lay, ws = method.last_layout, method.last_workspace
    P, H, E = shape.P, shape.H, shape.E
    I = sl.layer.w2_weight.shape[-1]  # the size the kernels see (a size that is no multiple of 64 is padded at load time)
    ids = _view(ws, lay.topk_ids, P, torch.int32).cpu().numpy().reshape(shape.M, shape.K)
    moe_index = _view(ws, lay.moe_index, P, torch.int32).cpu().numpy()
    lod = _view(ws, lay.lod, E + 1, torch.int32).cpu().numpy()
    R = P + (shape.M if shape.I_shared == I else 0)  # an equal-width shared expert adds rows [P, P+M)
    actq = _view(ws, lay.actq, R * I, torch.int8).cpu().numpy()
    if lay.codes_chunked:  # [I/64][R][64] -> [R][I]
        actq = actq.reshape(I // 64, R, 64).transpose(1, 0, 2)
    actq = np.ascontiguousarray(actq).reshape(R, I)[:P]
    topk_w = _view(ws, lay.topk_w, P, torch.float32).cpu().numpy().reshape(shape.M, shape.K)
    assert np.array_equal(ids, inter["topk_ids"]), "routing ids"
    assert np.array_equal(moe_index, inter["moe_index"]), "sorted token map"
    assert np.array_equal(lod, inter["lod"]), "lod"
    assert np.array_equal(topk_w.view(np.uint32), inter["topk_w"].view(np.uint32)), "routing weights"
    assert np.array_equal(actq, inter["actq"]), "int8 inputs of the down GEMM"
    assert np.array_equal(bits(out), ref_bits), "bf16 output vs C oracle"

    # the reference's torch expert loop, written independently of the C oracle
    w13, w13_max, w2, w2_max, shared = sl.host_weights()
    ref_t = tm.w8a8_moe(_host(sl.x), _host(sl.logits), w13, w13_max, w2, w2_max, shape.K, shape.scoring, True,
                        shape.n_group, shape.topk_group, shape.routed_scale, _host(sl.bias), shared, out_scale)
    assert rel_l2(out, ref_t) <= REL_L2_BF16


@pytest.mark.parametrize("hot,boost", [(1, 6.0), (3, 3.0)])
def test_skewed_decode_batches_match_oracles(hot, boost):
    """A few experts draw most tokens of a decode-sized batch: on the weight-streaming path they walk their rows in
    several 16-row passes (the launches that sort the pairs and quantise their rows themselves included), with and
    without a shared expert in the launches' tail."""
    from vllm_kunlun_amd import synth
    for base, over in (("qwen3-decode", dict(M=150, H=256, E=64, K=4, I=192)),
                       ("dsv3-decode", dict(M=80, H=256, E=32, K=4, I=128, n_group=4, topk_group=2, I_shared=128))):
        sl = synth.make_w8a8_layer(synth.scaled(synth.SHAPES[base], **over), "cuda", seed=hot)
        sl.logits[:, :hot] += boost
        _check_layer(sl)
        lod = _view(sl.layer.quant_method.last_workspace, sl.layer.quant_method.last_layout.lod, sl.shape.E + 1,
                    torch.int32).cpu().numpy()
        assert int(np.diff(lod).max()) > 32, "no expert with more than two passes of rows"
        assert sl.layer.quant_method.last_layout.codes_chunked, "not on the weight-streaming path"


def test_decode_launches_that_sort_and_quantise_keep_the_bits():
    """KMOE_SORT_IN_GEMM=0 / KMOE_QUANT_IN_GEMM=0 (read once per process, hence child processes) give the sort and
    the second quantisation launches of their own again: same output bits, same intermediates (int8 layers), same
    output bits (layers on packed 4-bit weights)."""
    import os
    import subprocess
    import sys
    code = r"""
import sys, zlib
sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[2])
import torch
from vllm_kunlun_amd import synth
for base, over in (("qwen3-decode", dict(M=64, H=512, E=128, K=8, I=768)),
                   ("dsv3-decode", dict(M=40, H=512, E=32, K=4, I=128, n_group=4, topk_group=2, I_shared=128))):
    sl = synth.make_w8a8_layer(synth.scaled(synth.SHAPES[base], **over), "cuda", seed=4)
    sl.logits[:, :2] += 2.0
    m = sl.layer.quant_method
    out = m.apply_monolithic(sl.layer, sl.x, sl.logits, **sl.apply_kwargs())
    torch.cuda.synchronize()
    lay, ws = m.last_layout, m.last_workspace
    P, E, I = sl.shape.P, sl.shape.E, sl.shape.I
    R = P + (sl.shape.M if sl.shape.I_shared == I else 0)
    parts = [out.view(torch.int16)] + [ws[o: o + n] for o, n in ((lay.moe_index, 4 * P), (lay.sorted_src, 4 * P),
             (lay.lod, 4 * (E + 1)), (lay.expert_m, 4 * E), (lay.actq, R * I), (lay.actmax, 4 * R))]
    print(*[zlib.crc32(t.cpu().numpy().tobytes()) for t in parts])
# packed 4-bit weights: the streaming kernel of that format sorts the pairs as well (16- and 32-row passes)
for M, E in ((64, 128), (40, 12)):
    shape = synth.scaled(synth.SHAPES["qwen3-decode"], M=M, H=256, E=E, K=4, I=128, quant="w4", group_size=128)
    sl = synth.make_layer(shape, "cuda", seed=5)
    sl.logits[:, :2] += 2.0
    out = sl.layer(sl.x, sl.logits)
    torch.cuda.synchronize()
    print(zlib.crc32(out.view(torch.int16).cpu().numpy().tobytes()))
"""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    sums = []
    for flag in ("1", "0"):
        env = dict(os.environ, KMOE_SORT_IN_GEMM=flag, KMOE_QUANT_IN_GEMM=flag)
        out = subprocess.run([sys.executable, "-c", code, root, os.path.join(root, "vllm-kunlun_amd")], env=env,
                             capture_output=True, text=True, timeout=110)
        assert out.returncode == 0, out.stderr[-2000:]
        sums.append(out.stdout.split())
    assert len(sums[0]) == 16 and sums[0] == sums[1], sums


def test_staged_ops_equal_fused():
    """The reference's op-by-op sequence through torch.ops._C.* gives the same bits."""
    from vllm_kunlun_amd import synth
    # P <= 768 and > 768; an intermediate size that is padded at load time
    for over in (dict(M=48, H=512, E=16, K=4, I=256), dict(M=200, H=256, E=8, K=4, I=128),
                 dict(M=48, H=512, E=16, K=4, I=96)):
        sl = synth.make_w8a8_layer(synth.scaled(synth.SHAPES["qwen3-decode"], **over), "cuda", seed=2)
        m = sl.layer.quant_method
        fused = m.apply_monolithic(sl.layer, sl.x, sl.logits)
        staged = m.apply_staged(sl.layer, sl.x, sl.logits)
        torch.cuda.synchronize()
        assert torch.equal(fused, staged)
    sl = synth.make_w8a8_layer(synth.scaled(synth.SHAPES["dsv3-decode"], M=40, H=512, E=32, K=4, I=128, n_group=4,
                                            topk_group=2, I_shared=0), "cuda", seed=3)
    m = sl.layer.quant_method
    kw = sl.apply_kwargs()
    fused = m.apply_monolithic(sl.layer, sl.x, sl.logits, **kw)
    staged = m.apply_staged(sl.layer, sl.x, sl.logits, **kw)
    torch.cuda.synchronize()
    assert torch.equal(fused, staged)


def test_tiled_and_rowmajor_weights_give_the_same_bits():
    """process_weights_after_loading tiles the int8 weights in place on the GPU; a layer
    kept row-major (tile_weights=False) must produce identical outputs, in the streaming
    regime (8 rows per expert) and in the tile kernel's (40 rows: 64-row tiles; 225 rows: 128-row tiles)."""
    from vllm_kunlun_amd import _plan, synth
    from vllm_kunlun_amd.quantization.compressed_tensors.compressed_tensors_moe import (
        KunlunCompressedTensorsW8A8Int8MoEMethod)
    for over in (dict(M=32, H=512, E=16, K=4, I=256), dict(M=160, H=512, E=16, K=4, I=256),
                 dict(M=900, H=256, E=8, K=2, I=128)):
        shape = synth.scaled(synth.SHAPES["dsv3-decode"], n_group=4, topk_group=2, I_shared=128, **over)
        tiled = synth.make_w8a8_layer(shape, "cuda", seed=9)
        assert _plan.is_tiled(tiled.layer.w13_weight) and _plan.is_tiled(tiled.shared[0])
        KunlunCompressedTensorsW8A8Int8MoEMethod.tile_weights = False
        try:
            plain = synth.make_w8a8_layer(shape, "cuda", seed=9)
        finally:
            del KunlunCompressedTensorsW8A8Int8MoEMethod.tile_weights
        assert not _plan.is_tiled(plain.layer.w13_weight)
        a = tiled.layer.quant_method.apply_monolithic(tiled.layer, tiled.x, tiled.logits, **tiled.apply_kwargs())
        assert tiled.layer.quant_method.last_layout.codes_chunked == (1 if over["M"] == 32 else 0)
        b = plain.layer.quant_method.apply_monolithic(plain.layer, plain.x, plain.logits, **plain.apply_kwargs())
        torch.cuda.synchronize()
        assert torch.equal(a, b)


@pytest.mark.parametrize("over", [dict(M=40, H=512, E=16, K=4, I=96), dict(M=700, H=256, E=8, K=2, I=160),
                                  dict(M=300, H=640, E=16, K=4, I=96, I_shared=96)],
                         ids=["96-stream", "160-tile-kernel", "96-shared-same-width"])
def test_padded_intermediate_size_keeps_every_bit(over):
    """An intermediate size that is no multiple of 64 is padded with zero channels at load time so that the
    weights can be tiled. The padded layer, the unpadded one (row-major kernels) and the oracle on the
    unpadded weights must agree bit for bit."""
    from vllm_kunlun_amd import _plan, synth
    from vllm_kunlun_amd.quantization.compressed_tensors.compressed_tensors_moe import (
        KunlunCompressedTensorsW8A8Int8MoEMethod)
    shape = synth.scaled(synth.SHAPES["dsv3-decode"], n_group=4, topk_group=2, **{"I_shared": 0, **over})
    padded = synth.make_w8a8_layer(shape, "cuda", seed=13)
    Ip = -(-shape.I // 64) * 64
    assert _plan.is_tiled(padded.layer.w13_weight) and padded.layer.w2_weight.shape[-1] == Ip
    assert padded.layer.intermediate_size_unpadded == shape.I
    KunlunCompressedTensorsW8A8Int8MoEMethod.pad_intermediate = False
    try:
        plain = synth.make_w8a8_layer(shape, "cuda", seed=13)
    finally:
        del KunlunCompressedTensorsW8A8Int8MoEMethod.pad_intermediate
    assert not _plan.is_tiled(plain.layer.w13_weight) and plain.layer.w2_weight.shape[-1] == shape.I
    a = padded.layer.quant_method.apply_monolithic(padded.layer, padded.x, padded.logits, **padded.apply_kwargs())
    b = plain.layer.quant_method.apply_monolithic(plain.layer, plain.x, plain.logits, **plain.apply_kwargs())
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    ref_bits = co.forward_w8a8(**_oracle_inputs(plain), out_scale=1.0)
    assert np.array_equal(bits(a), ref_bits), "padded layer vs C oracle on the unpadded weights"


def test_layer_forward_via_module_call():
    """FusedMoE.forward hands (layer, x, router_logits) to the method and the
    method picks the sigmoid/grouped parameters up from the layer attributes."""
    from vllm_kunlun_amd import synth
    sl = synth.make_w8a8_layer(synth.scaled(synth.SHAPES["dsv3-decode"], M=24, H=256, E=32, K=4, I=64, n_group=4,
                                            topk_group=2, I_shared=0), "cuda", seed=4)
    sl.layer.routed_scaling_factor = sl.shape.routed_scale
    a = sl.layer(sl.x, sl.logits)
    b = sl.layer.quant_method.apply_monolithic(sl.layer, sl.x, sl.logits, **sl.apply_kwargs())
    torch.cuda.synchronize()
    assert torch.equal(a, b)


def test_empty_batch():
    from vllm_kunlun_amd import synth
    sl = synth.make_w8a8_layer(synth.scaled(synth.SHAPES["qwen3-decode"], M=4, H=256, E=8, K=2, I=64), "cuda")
    out = sl.layer.quant_method.apply_monolithic(sl.layer, sl.x[:0], sl.logits[:0])
    assert out.shape == (0, 256)


ROUTER_CASES = [(1, 64, 8), (7, 256, 130), (64, 2048, 128), (128, 7168, 256), (300, 512, 384), (1100, 1024, 64)]


@pytest.mark.parametrize("M,H,E", ROUTER_CASES)
def test_router_gemm(M, H, E):
    """kmoe_router_gemm_bf16 through torch.ops._C.router_gemm_bf16_fp32 against the exact-sum oracle,
    within the f32 summation bound, and bit-identical from run to run (fixed plane order)."""
    import vllm_kunlun_amd  # noqa: F401
    torch.manual_seed(M + H + E)
    x = torch.randn(M, H).bfloat16()
    w = (torch.randn(E, H) * 0.05).bfloat16()
    ref, abs_sum = co.router_gemm(bits(x), bits(w))
    xd, wd = x.cuda(), w.cuda()
    got = torch.ops._C.router_gemm_bf16_fp32(xd, wd)
    again = torch.ops._C.router_gemm_bf16_fp32(xd, wd)
    torch.cuda.synchronize()
    assert torch.equal(got, again)
    err = np.abs(got.cpu().numpy() - ref)
    assert np.all(err <= H * 2.0 ** -24 * abs_sum + 1e-30), float(err.max())


@pytest.mark.parametrize("base,over", [("qwen3-decode", dict(M=40, H=256, E=64, K=4, I=128)),
                                       ("dsv3-decode", dict(M=48, H=512, E=32, K=4, I=256, n_group=4, topk_group=2,
                                                            I_shared=256)),
                                       ("qwen3-prefill", dict(M=1500, H=256, E=16, K=2, I=128))],
                         ids=["softmax", "sigmoid-shared", "many-tokens"])
def test_layer_with_the_router_inside(base, over):
    """apply_monolithic(router_logits=None, router_weight=W): the same bits as computing the logits
    with the stand-alone router GEMM and handing them in (the routing kernel adds the split-K planes
    in the order the reduction kernel does)."""
    from vllm_kunlun_amd import synth
    from vllm_kunlun_amd.ops.fused_moe.router import GateLinear
    shape = synth.scaled(synth.SHAPES[base], **over)
    sl = synth.make_w8a8_layer(shape, "cuda", seed=3)
    gate = GateLinear(shape.H, shape.E, device="cuda")
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    gate.weight.data.copy_((torch.randn(shape.E, shape.H, generator=g, device="cuda") * 0.05).bfloat16())
    logits, _ = gate(sl.x)
    m = sl.layer.quant_method
    kw = sl.apply_kwargs()
    ref = m.apply_monolithic(sl.layer, sl.x, logits, **kw)
    got = m.apply_monolithic(sl.layer, sl.x, None, router_weight=gate.weight, **kw)
    torch.cuda.synchronize()
    assert torch.equal(got, ref)


def test_layer_with_paced_tiles_gives_the_same_bits():
    """tile_variant = 12 (the m-tiles of one expert and channel block wait for each other so that they share
    the weight bytes in L2) only changes when workgroups run, and the wide 8-wave tiles (19, 18, 22: 128, 192, 256
    rows) only which workgroup computes a row: the output bits are those of the 128-row 4-wave tiles (6)."""
    from vllm_kunlun_amd import _lib as L
    from vllm_kunlun_amd import synth
    from vllm_kunlun_amd._plan import make_moe_plan
    # several m-tiles per expert (about 300 rows each) and a folded shared expert
    shape = synth.scaled(synth.SHAPES["dsv3-decode"], M=1200, H=512, E=16, K=4, I=256, n_group=4, topk_group=2,
                         I_shared=256)
    sl = synth.make_w8a8_layer(shape, "cuda", seed=12)
    lay = sl.layer
    outs = []
    for variant in (6, 0, 12, 12, 19, 18, 22, 17):
        out = torch.empty_like(sl.x)
        plan = make_moe_plan(L.KMOE_FMT_INT8, sl.x, sl.logits, out, shape.K, lay.w13_weight, lay.w2_weight,
                             lay.w13_weight_scale, lay.w2_weight_scale, shape.scoring, True, shape.n_group,
                             shape.topk_group, shape.routed_scale, sl.bias, sl.shared, 1.0, tile_variant=variant)
        plan()
        torch.cuda.synchronize()
        outs.append(out)
    assert all(torch.equal(outs[0], o) for o in outs[1:])
    oi = _oracle_inputs(sl)
    assert np.array_equal(bits(outs[1]), co.forward_w8a8(**oi))


@pytest.mark.parametrize("M", [48, 1500])
@pytest.mark.parametrize("scoring", ["softmax", "sigmoid"])
def test_int8_layer_as_an_expert_parallel_share(M, scoring):
    """kmoe_moe_forward with E_global / first_expert (the share of one expert-parallel rank: routing over all 32
    experts, the weights of 8 of them): bit for bit the oracle's stages on the pairs routed to the local experts,
    on the weight-streaming path (48 tokens) and on the tile kernel (1500), with grouped sigmoid routing and a
    correction bias over the global experts; pairs routed elsewhere add nothing."""
    from vllm_kunlun_amd import _lib as L, _plan
    from oracle import torch_moe as tm
    Eg, El, K, H, I = 32, 8, 4, 256, 128
    g = torch.Generator().manual_seed(M + len(scoring))
    x = (torch.randn(M, H, generator=g) * 1.5).bfloat16()
    logits = torch.randn(M, Eg, generator=g)
    bias = torch.randn(Eg, generator=g) * 0.1 if scoring == "sigmoid" else None
    route = dict(scoring_func=scoring, renormalize=True, num_expert_group=4 if scoring == "sigmoid" else None,
                 topk_group=2 if scoring == "sigmoid" else None, routed_scaling_factor=2.5 if scoring == "sigmoid" else 1.0,
                 e_score_correction_bias=None if bias is None else bias.cuda())
    w, ids = co._route(logits.numpy(), K, scoring, True, 4, 2, 2.5 if scoring == "sigmoid" else 1.0,
                       None if bias is None else bias.numpy())
    for rank in (0, 3):
        lo = rank * El
        gw = torch.Generator().manual_seed(100 + rank)
        w13q, s13 = tm.quantize_weight_per_channel((torch.randn(El * 2 * I, H, generator=gw) * 0.05))
        w2q, s2 = tm.quantize_weight_per_channel((torch.randn(El * H, I, generator=gw) * 0.05))
        w13q, w2q = w13q.view(El, 2 * I, H), w2q.view(El, H, I)
        w13_max, w2_max = (s13 * 127.0).view(El, 2 * I), (s2 * 127.0).view(El, H)
        d13, d2 = w13q.clone().cuda(), w2q.clone().cuda()
        assert _plan.tile_pair_(d13, d2)
        out = torch.empty(M, H, dtype=torch.bfloat16, device="cuda")
        plan = _plan.make_moe_plan(L.KMOE_FMT_INT8, x.cuda(), logits.cuda(), out, K, d13, d2, w13_max.cuda(),
                                   w2_max.cuda(), first_expert=lo, **route)
        plan()
        torch.cuda.synchronize()
        # the oracle's stages on the local pairs
        moe_index, src, _, lod = co.align(ids - np.int32(lo), El)
        xq, x_max = co.quant_i8_rows(bits(x))
        act, _ = co.grouped_gemm_i8(xq, x_max, w13q.numpy(), w13_max.numpy(), lod, act=1, row_src=src, src_div=K)
        aq, a_max = co.quant_i8_rows(act)
        down, _ = co.grouped_gemm_i8(aq, a_max, w2q.numpy(), w2_max.numpy(), lod)
        ref = co.combine(down, moe_index, w)
        assert np.array_equal(bits(out), ref), f"rank {rank}"
        assert 0 < int(lod[-1]) < M * K
        # the same share through the plugin method: the layer holds the rank's experts, method.moe names the rank
        from types import SimpleNamespace
        from vllm_kunlun_amd.quantization.compressed_tensors.compressed_tensors_moe import (
            KunlunCompressedTensorsW8A8Int8MoEMethod)
        method = KunlunCompressedTensorsW8A8Int8MoEMethod(moe=SimpleNamespace(experts_per_token=K, use_ep=True, ep_rank=rank))
        layer = SimpleNamespace(w13_weight=d13, w2_weight=d2, w13_weight_scale=w13_max.cuda(), w2_weight_scale=w2_max.cuda())
        kw = {k: v for k, v in route.items() if k != "renormalize"}
        out2 = method.apply_monolithic(layer, x.cuda(), logits.cuda(), **kw)
        torch.cuda.synchronize()
        assert torch.equal(out2, out)
