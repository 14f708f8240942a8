"""GPU parity of the unquantized (bf16) and fp8 block-scaled paths.

MFMA accumulates f32 in the hardware's own order, so these are held to the
north-star tolerances instead of bit equality: bf16 outputs rel-L2 <= 1e-2,
fp8 rel-L2 <= 3e-2 — against the C oracle (sequential f32 sums) and against the
torch oracle. The fp8 path has no counterpart in the reference: its parity is
with this repository's own oracle only (DeepSeek-V3 block-scale recipe).
"""
import numpy as np
import pytest
import torch

from conftest import bits, from_bits, rel_l2

pytestmark = pytest.mark.gpu

from oracle import c_oracle as co  # noqa: E402
from oracle import torch_moe as tm  # noqa: E402

REL_L2_BF16 = 1e-2
REL_L2_FP8 = 3e-2


@pytest.fixture(scope="module")
def L():
    from vllm_kunlun_amd import _lib
    return _lib


def _lod(counts):
    return np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)


CASES = [
    (1, 64, 128, [16]),
    (4, 64, 256, [3, 0, 17, 1]),
    (3, 96, 776, [5, 40, 7]),      # k*2 bytes not a multiple of the 256-byte chunk
    (2, 256, 1024, [130, 129]),
    (8, 128, 64, [4, 4, 0, 9, 33, 1, 0, 2]),
]


BF16_TILED_CASES = [
    (1, 64, 128, [16]),
    (4, 64, 256, [3, 0, 17, 1]),
    (2, 256, 1024, [130, 129]),
    (3, 96, 320, [5, 140, 7]),                                    # 5 chunks of 128 bytes
    (8, 128, 64, [4, 4, 0, 9, 33, 1, 0, 2]),
    (20, 1024, 128, [((53 * i) % 300) for i in range(20)]),       # several tiles per workgroup walk
    # an odd number of 64-byte steps (k % 64 == 32): the half chunk at every position of the ring
    (3, 64, 96, [1, 260, 17]),
    (2, 96, 160, [140, 3]),
    (4, 128, 224, [70, 0, 129, 5]),
    (2, 64, 288, [33, 200]),
]


@pytest.mark.parametrize("E,n,k,counts", BF16_TILED_CASES)
@pytest.mark.parametrize("variant", [1, 2, 3, 5, 6, 11])
@pytest.mark.parametrize("act", [0, 1])
def test_grouped_gemm_bf16_tiled_weights(L, E, n, k, counts, variant, act):
    """bf16 weights re-arranged (as bytes) by kmoe_tile_weights_i8: the LDS-staged kernels (1-3) and
    the persistent tile kernel (5: tile height from the rows per expert; 6: 128 rows; 11: 64 rows)."""
    _bf16_case(L, E, n, k, counts, variant, act, tiled=True)


def test_grouped_gemm_bf16_half_chunk_ignores_the_repeated_step(L):
    """With an odd number of 64-byte steps the tile kernel's last chunk holds the step before the last a
    second time; it must count as zeros whatever it holds. An infinite activation there gives +-inf in every
    channel (as in the exact product), never NaN."""
    E, n, k, rows = 1, 64, 96, 70
    torch.manual_seed(5)
    a = torch.randn(rows, k).bfloat16()
    a[3, 40] = float("inf")  # element 40: in the second step, which the half chunk reads again
    w = (torch.randn(E, n, k) * 0.05).bfloat16()
    w[w == 0] = 0.05
    da, dw = a.cuda(), w.cuda()
    dt = torch.empty_like(dw)
    L.check(L.lib.kmoe_tile_weights_i8(dw.data_ptr(), dt.data_ptr(), E, n, 2 * k, L.stream()))
    dl = torch.tensor([0, rows], dtype=torch.int32, device="cuda")
    y = torch.zeros(rows, n, dtype=torch.bfloat16, device="cuda")
    g = L.GemmBf16Args()
    g.a, g.lda, g.src_div, g.w, g.lod = da.data_ptr(), k, 1, dt.data_ptr(), dl.data_ptr()
    g.E, g.n, g.k, g.rows = E, n, k, rows
    g.y, g.ldy, g.act, g.variant, g.w_layout = y.data_ptr(), n, 0, 5, L.KMOE_W_TILED
    L.check(L.lib.kmoe_grouped_gemm_bf16(g, L.stream()))
    torch.cuda.synchronize()
    y = y.float().cpu()
    assert not torch.isnan(y).any()
    assert torch.equal(y[3], torch.sign(w[0, :, 40].float()) * float("inf"))
    keep = [r for r in range(rows) if r != 3]
    assert rel_l2(y[keep], a[keep].float() @ w[0].float().T) <= 2e-3


@pytest.mark.parametrize("E,n,k,counts", CASES)
@pytest.mark.parametrize("variant", [1, 2, 3])
@pytest.mark.parametrize("act", [0, 1])
def test_grouped_gemm_bf16(L, E, n, k, counts, variant, act):
    _bf16_case(L, E, n, k, counts, variant, act, tiled=False)


def _bf16_case(L, E, n, k, counts, variant, act, tiled):
    torch.manual_seed(E * n + k)
    lod = _lod(counts)
    rows = int(lod[-1])
    a = torch.randn(rows, k).bfloat16()
    w = (torch.randn(E, n, k) * 0.05).bfloat16()
    ref = co.grouped_gemm_bf16(bits(a), bits(w), lod, act=act)
    n_out = n // 2 if act else n
    da, dw, dl = a.cuda(), w.cuda(), torch.from_numpy(lod).cuda()
    y = torch.zeros(rows, n_out, dtype=torch.bfloat16, device="cuda")
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
    L.check(L.lib.kmoe_grouped_gemm_bf16(g, L.stream()))
    torch.cuda.synchronize()
    assert rel_l2(y, from_bits(ref)) <= 2e-3   # well inside the 1e-2 bar: only summation order differs
    # independent torch check of one expert
    e = int(np.argmax(counts))
    r0, r1 = lod[e], lod[e + 1]
    t = a[r0:r1].float() @ w[e].float().T
    if act:
        t = tm.silu_and_mul(t.bfloat16()).float()
    assert rel_l2(y[r0:r1], t) <= REL_L2_BF16


FP8_CASES = [
    (1, 128, 128, [16]),
    (3, 256, 384, [5, 0, 21]),
    (2, 512, 1024, [70, 3]),
]


FP8_TILED_CASES = FP8_CASES + [
    (2, 256, 640, [140, 3]),                                      # odd number of 128-byte chunks
    (20, 1024, 256, [((53 * i) % 300) for i in range(20)]),       # several tiles per workgroup walk
    (5, 256, 384, [192, 193, 0, 256, 257]),                       # ends of the 8-wave tiles (192 and 256 rows)
    (6, 256, 384, [140, 150, 135, 160, 145, 138]),                # variant 17: the 192-row tiles are chosen on the device,
    (8, 256, 256, [300, 10, 290, 20, 310, 15, 150, 100]),         # ... and here the 128-row tiles
]


@pytest.mark.parametrize("E,n,k,counts", FP8_TILED_CASES)
@pytest.mark.parametrize("variant", [1, 2, 3, 5, 6, 8, 11, 13, 14, 17, 18, 19])
@pytest.mark.parametrize("act", [0, 1])
def test_grouped_gemm_fp8_block_tiled_weights(L, E, n, k, counts, variant, act):
    """The same product with the weight bytes re-arranged by kmoe_tile_weights_i8: the LDS-staged
    kernels (1-3) and the persistent tile kernel (5: tile height by the rows per expert; 6: 128; 11: 64; 13: 96 rows;
    14, 8: 8-wave tiles of 192 and 256 rows; 17: 192- or 128-row tiles, decided on the device; 18, 19: wide tiles
    of 192 and 128 rows on the asynchronous activation path, rows past a tile's end skipped)."""
    _fp8_case(L, E, n, k, counts, variant, act, tiled=True)


@pytest.mark.parametrize("E,n,k,counts", FP8_TILED_CASES)
@pytest.mark.parametrize("variant,tiled", [(1, False), (2, True), (5, True), (6, True), (11, True), (12, True), (13, True),
                                           (14, True), (8, True), (17, True), (18, True), (19, True)])
@pytest.mark.parametrize("act", [0, 1])
def test_grouped_gemm_fp8_block_half_results(L, E, n, k, counts, variant, tiled, act):
    """act_dtype = KMOE_DT_F16: the LDS-staged kernel and the tile kernel's 64-row, 128-row and paced shapes."""
    _fp8_case(L, E, n, k, counts, variant, act, tiled=tiled, half=True)


@pytest.mark.parametrize("E,n,k,counts", FP8_CASES)
@pytest.mark.parametrize("variant", [1, 2, 3])
@pytest.mark.parametrize("act", [0, 1])
def test_grouped_gemm_fp8_block(L, E, n, k, counts, variant, act):
    _fp8_case(L, E, n, k, counts, variant, act, tiled=False)


def _fp8_case(L, E, n, k, counts, variant, act, tiled, half=False):
    if act and n % 256:
        pytest.skip("SwiGLU needs n % 256 == 0 for block scales")
    torch.manual_seed(E * n + k + 1)
    lod = _lod(counts)
    rows = int(lod[-1])
    x = (torch.randn(rows, k) * 2).bfloat16()
    xq, xs = tm.quant_fp8_group128(x)
    wq, ws = tm.quantize_weight_fp8_block128(torch.randn(E, n, k) * 0.02)
    a8, w8 = xq.view(torch.uint8), wq.view(torch.uint8)
    ref = co.grouped_gemm_fp8(a8.numpy(), xs.numpy(), w8.numpy(), ws.numpy(), lod, act=act, f16=half)
    n_out = n // 2 if act else n
    da, ds, dw, dws, dl = a8.cuda(), xs.contiguous().cuda(), w8.cuda(), ws.contiguous().cuda(), torch.from_numpy(lod).cuda()
    y = torch.zeros(rows, n_out, dtype=torch.float16 if half else torch.bfloat16, device="cuda")
    g = L.GemmFp8Args()
    g.act_dtype = L.KMOE_DT_F16 if half else L.KMOE_DT_BF16
    if tiled:
        dt = torch.empty_like(dw)
        L.check(L.lib.kmoe_tile_weights_i8(dw.data_ptr(), dt.data_ptr(), E, n, k, L.stream()))
        dw = dt
        g.w_layout = L.KMOE_W_TILED
    g.a, g.lda, g.a_scale, g.src_div = da.data_ptr(), k, ds.data_ptr(), 1
    g.w, g.w_scale, g.lod = dw.data_ptr(), dws.data_ptr(), dl.data_ptr()
    g.E, g.n, g.k, g.rows = E, n, k, rows
    g.y, g.ldy, g.act, g.variant = y.data_ptr(), n_out, act, variant
    L.check(L.lib.kmoe_grouped_gemm_fp8_block(g, L.stream()))
    torch.cuda.synchronize()
    if half:  # results (and gate and up before SiLU-mul) rounded to IEEE half
        assert rel_l2(y, torch.from_numpy(ref.view(np.float16).copy())) <= 2e-3
        return
    assert rel_l2(y, from_bits(ref)) <= 2e-3
    if not act:  # torch restatement of the block-scaled product, one expert
        e = int(np.argmax(counts))
        r0, r1 = lod[e], lod[e + 1]
        t = tm.fp8_block_gemm(xq[r0:r1], xs[r0:r1], wq[e], ws[e])
        assert rel_l2(y[r0:r1], t) <= REL_L2_FP8


def _host(t):
    return None if t is None else t.detach().cpu()


def test_bf16_layer_config1_and_variants():
    """The small unquantized configuration (32 tokens, hidden 512, 8 experts, top-2 softmax, I=256, bf16)
    through FusedMoE -> KunlunUnquantizedFusedMoEMethod.apply_monolithic -> KunlunOps.fused_moe."""
    from vllm_kunlun_amd import synth
    for shape in (synth.SHAPES["tiny-bf16"],
                  synth.scaled(synth.SHAPES["tiny-bf16"], M=300, H=256, E=16, K=4, I=128),
                  synth.scaled(synth.SHAPES["tiny-bf16"], M=150, H=96, E=16, K=4, I=96),  # 192-byte rows tile
                  synth.scaled(synth.SHAPES["dsv3-decode"], M=40, H=256, E=32, K=4, I=128, n_group=4, topk_group=2,
                               I_shared=0, quant="none")):
        sl = synth.make_bf16_layer(shape, "cuda", seed=5)
        out = sl.layer(sl.x, sl.logits)
        torch.cuda.synchronize()
        w13, _, w2, _, _ = sl.host_weights()  # row-major copies of the (tiled) device weights
        ref = co.forward_bf16(bits(sl.x), _host(sl.logits).numpy(), bits(w13), bits(w2), shape.K,
                              shape.scoring, True, shape.n_group, shape.topk_group, 1.0,
                              None if sl.bias is None else _host(sl.bias).numpy())
        assert rel_l2(out, from_bits(ref)) <= REL_L2_BF16
        if shape.scoring == "softmax":  # the reference's own torch loop (fused_moe_ep)
            ref_t = tm.bf16_moe(_host(sl.x), _host(sl.logits), w13, w2, shape.K,
                                True)
            assert rel_l2(out, ref_t) <= REL_L2_BF16


def test_bf16_golden_fixture_and_ep_entry():
    import os
    from vllm_kunlun_amd.ops._kunlun_ops import KunlunOps
    g = dict(np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "bf16_tiny_layer.npz")))
    x, w13, w2 = (from_bits(g[k]).cuda() for k in ("x", "w13", "w2"))
    logits = torch.from_numpy(g["logits"]).cuda()
    out = KunlunOps.fused_moe_ep(x, w13, w2, logits, 0, int(g["K"]), True)
    out2 = KunlunOps.fused_moe(x, w13, w2, logits, 0, int(g["K"]), True)
    torch.cuda.synchronize()
    assert rel_l2(out, from_bits(g["out"])) <= REL_L2_BF16
    assert torch.equal(out, out2)
    with pytest.raises(ValueError):  # a rank beyond 0 needs logits over more experts than the weights hold
        KunlunOps.fused_moe_ep(x, w13, w2, logits, 1, int(g["K"]), True)


@pytest.mark.parametrize("M,renormalize", [(24, True), (24, False), (700, True)])
def test_fused_moe_ep_shares(M, renormalize):
    """KunlunOps.fused_moe_ep as an expert-parallel rank calls it (ops/_kunlun_ops.py:640-696): logits over all 16
    experts, the weights of 4 of them, ep_rank = 0..3. Every share against the oracle's share and against the
    reference's loop restated in torch; a token none of whose experts are local gets exact zeros; the shares add
    up to the layer's output (what the ranks' all-reduce makes)."""
    from vllm_kunlun_amd.ops._kunlun_ops import KunlunOps
    from vllm_kunlun_amd import _plan
    Eg, El, K, H, I = 16, 4, 4, 256, 128
    g = torch.Generator().manual_seed(M)
    x = torch.randn(M, H, generator=g).bfloat16()
    logits = torch.randn(M, Eg, generator=g)
    w13 = (torch.randn(Eg, 2 * I, H, generator=g) * 0.05).bfloat16()
    w2 = (torch.randn(Eg, H, I, generator=g) * 0.05).bfloat16()
    _, ids = co.softmax_topk(logits.numpy(), K, renormalize)
    total = torch.zeros(M, H, dtype=torch.float64)
    for rank in range(Eg // El):
        lo = rank * El
        w13_r, w2_r = w13[lo:lo + El].contiguous().cuda(), w2[lo:lo + El].contiguous().cuda()
        if rank % 2:  # tiled local weights as the method keeps them, row-major ones as a caller may hand them over
            assert _plan.tile_pair_(w13_r, w2_r)
        out = KunlunOps.fused_moe_ep(x.cuda(), w13_r, w2_r, logits.cuda(), rank, K, renormalize)
        torch.cuda.synchronize()
        ref = co.forward_bf16(bits(x), logits.numpy(), bits(w13[lo:lo + El]), bits(w2[lo:lo + El]), K, "softmax",
                              renormalize, first_expert=lo)
        assert rel_l2(out, from_bits(ref)) <= REL_L2_BF16
        assert rel_l2(out, tm.bf16_moe(x, logits, w13[lo:lo + El], w2[lo:lo + El], K, renormalize, ep_rank=rank)) <= REL_L2_BF16
        elsewhere = ~((ids >= lo) & (ids < lo + El)).any(1)
        assert elsewhere.any() or M > 100
        assert not out.cpu()[torch.from_numpy(elsewhere)].any()
        total += out.cpu().double()
    whole = tm.bf16_moe(x, logits, w13, w2, K, renormalize)
    assert rel_l2(total, whole) <= REL_L2_BF16


def test_moe_fc_op_bf16_swish_glu():
    """The operator-level bf16 call with act="SWISH_GLU": result in the first half of y's columns
    (reference use: ops/_kunlun_ops.py:595-606)."""
    import vllm_kunlun_amd  # noqa: F401
    torch.manual_seed(0)
    E, n, k = 4, 128, 256
    counts = [10, 0, 33, 5]
    lod = torch.from_numpy(_lod(counts)).cuda()
    rows = sum(counts)
    x = torch.randn(rows, k).bfloat16().cuda()
    w = (torch.randn(E, n, k) * 0.05).bfloat16().cuda()
    y = torch.zeros(rows, 1, n, dtype=torch.bfloat16, device="cuda")
    idx = torch.arange(rows, dtype=torch.int32, device="cuda")
    torch.ops._C.moe_fc(x, w, lod, idx, 1, y, "SWISH_GLU")
    torch.cuda.synchronize()
    ref = co.grouped_gemm_bf16(bits(x), bits(w), lod.cpu().numpy(), act=1)
    assert rel_l2(y.view(rows, n)[:, : n // 2], from_bits(ref)) <= 2e-3
    assert torch.all(y.view(rows, n)[:, n // 2:] == 0)


@pytest.mark.parametrize("E,n,k,counts,tail", [(3, 256, 384, [5, 0, 21], 40), (2, 512, 1024, [70, 3], 7),
                                               (20, 1024, 256, [((53 * i) % 300) for i in range(20)], 300),
                                               (2, 256, 128, [0, 0], 33)])
@pytest.mark.parametrize("variant", [0, 1, 2, 3, 5, 6, 11, 13, 18, 19])
@pytest.mark.parametrize("act", [0, 1])
def test_grouped_gemm_fp8_block_tail_expert(L, E, n, k, counts, tail, variant, act):
    """w_tail / w_scale_tail: one more expert in the same launch, whose `tail` rows follow the routed
    rows and read activation rows tail_src0 + i (a shared expert folded into the routed GEMM). The
    oracle runs it as expert E of a weight tensor with E + 1 experts."""
    torch.manual_seed(E * n + k + tail + act)
    lod = _lod(counts)
    rows = int(lod[-1])
    lod_all = np.concatenate([lod, [rows + tail]]).astype(np.int32)
    x = (torch.randn(rows + tail, k) * 2).bfloat16()
    xq, xs = tm.quant_fp8_group128(x)
    wq, ws = tm.quantize_weight_fp8_block128(torch.randn(E + 1, n, k) * 0.02)
    a8, w8 = xq.view(torch.uint8), wq.view(torch.uint8)
    ref = co.grouped_gemm_fp8(a8.numpy(), xs.numpy(), w8.numpy(), ws.numpy(), lod_all, act=act)
    n_out = n // 2 if act else n
    da, ds, dws = a8.cuda(), xs.contiguous().cuda(), ws.contiguous().cuda()
    dl = torch.from_numpy(lod).cuda()
    dw, dwt = torch.empty(E, n, k, dtype=torch.uint8, device="cuda"), torch.empty(1, n, k, dtype=torch.uint8, device="cuda")
    L.check(L.lib.kmoe_tile_weights_i8(w8[:E].contiguous().cuda().data_ptr(), dw.data_ptr(), E, n, k, L.stream()))
    L.check(L.lib.kmoe_tile_weights_i8(w8[E:].contiguous().cuda().data_ptr(), dwt.data_ptr(), 1, n, k, L.stream()))
    y = torch.zeros(rows + tail, n_out, dtype=torch.bfloat16, device="cuda")
    g = L.GemmFp8Args()
    g.w_layout = L.KMOE_W_TILED
    g.a, g.lda, g.a_scale, g.src_div = da.data_ptr(), k, ds.data_ptr(), 1
    g.w, g.w_scale, g.lod = dw.data_ptr(), dws[:E].contiguous().data_ptr(), dl.data_ptr()
    ws_tail = dws[E].contiguous()
    g.w_tail, g.w_scale_tail = dwt.data_ptr(), ws_tail.data_ptr()
    g.tail_row0, g.tail_rows, g.tail_src0 = rows, tail, rows
    g.E, g.n, g.k, g.rows = E, n, k, rows
    g.y, g.ldy, g.act, g.variant = y.data_ptr(), n_out, act, variant
    L.check(L.lib.kmoe_grouped_gemm_fp8_block(g, L.stream()))
    torch.cuda.synchronize()
    want = from_bits(ref)
    assert rel_l2(y[:rows], want[:rows]) <= 2e-3 if rows else True
    assert rel_l2(y[rows:], want[rows:]) <= 2e-3


FP8_LAYERS = [
    ("fp8-softmax", "qwen3-decode", dict(M=40, H=256, E=16, K=4, I=128)),
    ("fp8-dsv3-shared", "dsv3-decode", dict(M=48, H=512, E=32, K=4, I=256, n_group=4, topk_group=2, I_shared=128)),
    ("fp8-kimi-many-rows", "kimi-decode", dict(M=400, H=256, E=24, K=8, I=128, I_shared=0)),
    # a shared expert of the routed experts' width: a pass of its own at 5 rows per expert; inside the routed
    # launches as one more expert at 30 (64-row tiles) and 175 rows per expert (128-row tiles)
    ("fp8-shared-same-width-few-rows", "dsv3-decode", dict(M=40, H=512, E=32, K=4, I=128, n_group=4, topk_group=2,
                                                       I_shared=128)),
    ("fp8-shared-folded-short-tiles", "dsv3-decode", dict(M=120, H=256, E=8, K=2, I=128, n_group=2, topk_group=1,
                                                          I_shared=128)),
    ("fp8-shared-folded-tall-tiles", "dsv3-decode", dict(M=700, H=256, E=8, K=2, I=128, n_group=2, topk_group=1,
                                                         I_shared=128)),
]


@pytest.mark.parametrize("name,base,over", FP8_LAYERS, ids=[c[0] for c in FP8_LAYERS])
def test_fp8_layer(name, base, over):
    from vllm_kunlun_amd import synth
    shape = synth.scaled(synth.SHAPES[base], quant="fp8", **over)
    sl = synth.make_fp8_layer(shape, "cuda", seed=6)
    m = sl.layer.quant_method
    out = m.apply_monolithic(sl.layer, sl.x, sl.logits, **sl.apply_kwargs())
    torch.cuda.synchronize()
    u8 = lambda t: _host(t).view(torch.uint8).numpy()  # noqa: E731
    w13, w13_s, w2, w2_s, sh = sl.host_weights()  # row-major copies of the (tiled) device weights
    shared = None
    if sh is not None:
        shared = (u8(sh[0]), sh[1].numpy(), u8(sh[2]), sh[3].numpy())
    ref = co.forward_fp8(bits(sl.x), _host(sl.logits).numpy(), u8(w13), w13_s.numpy(),
                         u8(w2), w2_s.numpy(), shape.K, shape.scoring, True,
                         shape.n_group, shape.topk_group, shape.routed_scale,
                         None if sl.bias is None else _host(sl.bias).numpy(), shared)
    assert rel_l2(out, from_bits(ref)) <= REL_L2_FP8
    # routing and sort are format-independent: still bit-exact
    P = shape.P
    ids = m.last_workspace[m.last_layout.topk_ids: m.last_layout.topk_ids + 4 * P].view(torch.int32).cpu().numpy()
    w_ref, ids_ref = (co.softmax_topk(_host(sl.logits).numpy(), shape.K, True) if shape.scoring == "softmax" else
                      co.sigmoid_group_topk_norm(_host(sl.logits).numpy(), _host(sl.bias).numpy(), shape.K,
                                                 shape.n_group, shape.topk_group, shape.routed_scale))
    assert np.array_equal(ids.reshape(shape.M, shape.K), ids_ref)


@pytest.mark.parametrize("E,n,k,counts", [(1, 64, 128, [16]), (4, 128, 256, [3, 0, 17, 40]), (3, 96, 776, [5, 40, 7]),
                                          (2, 544, 320, [140, 3]), (20, 512, 128, [((53 * i) % 300) for i in range(20)])])
@pytest.mark.parametrize("act", [0, 2])
@pytest.mark.parametrize("tiled,variant", [(False, 0), (True, 0), (True, 1), (True, 5), (True, 6), (True, 11)])
def test_grouped_gemm_bf16_bias_and_swigluoai(L, E, n, k, counts, act, tiled, variant):
    """The expert-bias branch of the bf16 GEMM: y = bf16(bf16(a.w^T) + bias), act 2 = gpt-oss activation;
    on the LDS-staged kernels and (tiled weights; variants 5, 6, 11 force it) on the persistent tile kernel,
    whose epilogue adds the bias and pairs the interleaved gate/up columns."""
    if tiled and (2 * k) % 64:
        pytest.skip("tiled weights need 64 bytes of K")
    if not tiled and E >= 20:
        pytest.skip("large case: tiled weights only")
    torch.manual_seed(E + n + k + act)
    lod = _lod(counts)
    rows = int(lod[-1])
    a = torch.randn(rows, k).bfloat16()
    w = (torch.randn(E, n, k) * 0.05).bfloat16()
    b = (torch.randn(E, n) * 0.3).bfloat16()
    ref = co.grouped_gemm_bf16_bias(bits(a), bits(w), bits(b), lod, act=act)
    n_out = n // 2 if act else n
    da, dw, db, dl = a.cuda(), w.cuda(), b.cuda(), torch.from_numpy(lod).cuda()
    y = torch.zeros(rows, n_out, dtype=torch.bfloat16, device="cuda")
    g = L.GemmBf16Args()
    if tiled:
        dt = torch.empty_like(dw)
        L.check(L.lib.kmoe_tile_weights_i8(dw.data_ptr(), dt.data_ptr(), E, n, 2 * k, L.stream()))
        dw = dt
        g.w_layout = L.KMOE_W_TILED
    g.a, g.lda, g.src_div = da.data_ptr(), k, 1
    g.w, g.lod, g.bias = dw.data_ptr(), dl.data_ptr(), db.data_ptr()
    g.E, g.n, g.k, g.rows = E, n, k, rows
    g.y, g.ldy, g.act, g.act_alpha, g.act_limit = y.data_ptr(), n_out, act, 1.702, 7.0
    g.variant = variant
    L.check(L.lib.kmoe_grouped_gemm_bf16(g, L.stream()))
    torch.cuda.synchronize()
    assert rel_l2(y, from_bits(ref)) <= 3e-3
    g.act = 1  # SwiGLU with a bias is not a path of the reference
    with pytest.raises(NotImplementedError):
        L.check(L.lib.kmoe_grouped_gemm_bf16(g, L.stream()))


def test_swigluoai_op_is_the_oracle_sequence():
    import vllm_kunlun_amd  # noqa: F401
    torch.manual_seed(2)
    y = (torch.randn(37, 64) * 4).bfloat16()
    got = torch.ops._C.swigluoai_and_mul(y.cuda())
    torch.cuda.synchronize()
    assert np.array_equal(bits(got), co.swigluoai_and_mul(bits(y)))


@pytest.mark.parametrize("M,tiled", [(70, False), (70, True), (600, True)])
def test_fused_moe_expert_bias_branch(M, tiled):
    """KunlunOps.fused_moe(..., w1_bias, w2_bias): the gpt-oss branch (ops/_kunlun_ops.py:433-468) against the
    C oracle and the reference's torch loop restated; row-major weights, and tiled weights at 35 (64-row tiles)
    and 300 rows per expert (128-row tiles) on the tile kernel."""
    from vllm_kunlun_amd import _plan
    from vllm_kunlun_amd.ops._kunlun_ops import KunlunOps
    torch.manual_seed(4)
    H, E, K, I = 128, 8, 4, 64
    x = torch.randn(M, H).bfloat16()
    logits = torch.randn(M, E)
    w13 = (torch.randn(E, 2 * I, H) * 0.1).bfloat16()
    w2 = (torch.randn(E, H, I) * 0.1).bfloat16()
    b13 = (torch.randn(E, 2 * I) * 0.2).bfloat16()
    b2 = (torch.randn(E, H) * 0.2).bfloat16()
    w13d, w2d = w13.cuda(), w2.cuda()
    if tiled:
        assert _plan.tile_pair_(w13d, w2d)
    out = KunlunOps.fused_moe(x.cuda(), w13d, w2d, logits.cuda(), 0, K, True, w1_bias=b13.cuda(),
                              w2_bias=b2.cuda())
    torch.cuda.synchronize()
    ref = from_bits(co.forward_bf16(bits(x), logits.numpy(), bits(w13), bits(w2), K, w13_bias=bits(b13),
                                    w2_bias=bits(b2)))
    assert rel_l2(out, ref) <= REL_L2_BF16
    assert rel_l2(out, tm.bf16_moe_bias(x, logits, w13, w2, b13, b2, K)) <= REL_L2_BF16


@pytest.mark.parametrize("group_size", [None, 32])
def test_w4a16_method_unpacks_once_and_runs_the_bf16_path(group_size):
    """KunlunCompressedTensorsWNA16MoEMethod: packed 4-bit weights -> bf16 (kmoe_dequant_w4_bf16, bit-exact
    vs the oracle) -> tiled -> KunlunOps.fused_moe; output against the C oracle on the unpacked weights."""
    from vllm_kunlun_amd.ops.fused_moe.layer import FusedMoE
    from vllm_kunlun_amd.quantization.compressed_tensors.compressed_tensors import CompressedTensorsConfig
    from vllm_kunlun_amd.quantization.compressed_tensors.compressed_tensors_moe import (
        KunlunCompressedTensorsMoEMethod, KunlunCompressedTensorsWNA16MoEMethod)
    from vllm_kunlun_amd._plan import rowmajor_int8_weights
    weights = {"num_bits": 4, "type": "int", "symmetric": True, "dynamic": False,
               "strategy": "group" if group_size else "channel", "group_size": group_size}
    cfg = CompressedTensorsConfig.from_config({"quant_method": "compressed-tensors", "format": "pack-quantized",
                                               "config_groups": {"g": {"targets": ["Linear"], "weights": weights,
                                                                       "input_activations": None,
                                                                       "format": "pack-quantized"}}})
    E, H, I, M, K = 8, 128, 64, 50, 2
    stub = FusedMoE(num_experts=E, top_k=K, hidden_size=H, intermediate_size=I)
    method = KunlunCompressedTensorsMoEMethod.get_moe_method(cfg, stub, "m.experts")
    assert isinstance(method, KunlunCompressedTensorsWNA16MoEMethod)
    layer = FusedMoE(num_experts=E, top_k=K, hidden_size=H, intermediate_size=I, quant_method=method, device="cuda")
    g = torch.Generator().manual_seed(9)
    ckpt = {}
    for e in range(E):
        for proj, (n, k) in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I))):
            ckpt[f"m.experts.{e}.{proj}.weight_packed"] = torch.randint(0, 256, (n, k // 2), generator=g, dtype=torch.uint8)
            ckpt[f"m.experts.{e}.{proj}.weight_scale"] = (torch.rand(n, k // group_size if group_size else 1,
                                                                      generator=g) * 0.02 + 0.002).bfloat16()
    assert len(layer.load_weights(ckpt.items())) == 6 * E
    packed13, scale13 = layer.w13_weight_packed.data.cpu(), layer.w13_weight_scale.data.cpu()
    packed2, scale2 = layer.w2_weight_packed.data.cpu(), layer.w2_weight_scale.data.cpu()
    method.process_weights_after_loading(layer)
    assert not hasattr(layer, "w13_weight_packed")
    w13 = rowmajor_int8_weights(layer.w13_weight).cpu()
    w2 = rowmajor_int8_weights(layer.w2_weight).cpu()
    assert np.array_equal(bits(w13), co.dequant_w4_bf16(packed13.numpy(), bits(scale13), group_size or H))
    assert np.array_equal(bits(w2), co.dequant_w4_bf16(packed2.numpy(), bits(scale2), group_size or I))
    gx = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(M, H, generator=gx, device="cuda").bfloat16()
    logits = torch.randn(M, E, generator=gx, device="cuda")
    out = layer(x, logits)
    torch.cuda.synchronize()
    ref = co.forward_bf16(bits(x), logits.cpu().numpy(), bits(w13), bits(w2), K)
    assert rel_l2(out, from_bits(ref)) <= REL_L2_BF16


W4_CASES = [
    # E, n, k, rows per expert, group size (None: one scale per row)
    (1, 64, 128, [16], 128),
    (4, 64, 256, [3, 0, 17, 1], 32),
    (3, 96, 384, [5, 40, 7], 128),
    (8, 256, 1024, [4, 4, 0, 9, 33, 1, 0, 2], 64),
    (2, 128, 512, [70, 3], None),
    (16, 1536, 256, [(5 * i) % 11 for i in range(16)], 128),
    (3, 96, 384, [5, 40, 7], 96),      # a group of 3 x 32 values: the group index is a division, not a shift
    (2, 64, 4224, [5, 20], 32),        # 132 groups per channel: too many for the LDS copy, scales read from memory
    (3, 96, 384, [130, 0, 260], 128),  # experts of two and three 128-row tiles, an empty one between them
    (5, 320, 256, [128, 1, 0, 129, 64], 64),  # tiles that end exactly at an expert's last row, and one row past it
    (6, 64, 256, [64, 65, 96, 97, 0, 192], 128),  # the same for the 64- and 96-row tiles
]


@pytest.mark.parametrize("E,n,k,counts,gs", W4_CASES)
@pytest.mark.parametrize("variant", [0, 1, 2, 4, 8, 64, 96, 128])
@pytest.mark.parametrize("act", [0, 1])
@pytest.mark.parametrize("gather,frag16", [(False, False), (True, False), (True, True)])
def test_grouped_gemm_w4a16(L, E, n, k, counts, gs, variant, act, gather, frag16):
    """Packed 4-bit weights unpacked in registers (variants 1, 2, 4: the streaming kernel; 64, 96, 128 and its
    older name 8: the tile kernel with tiles of that many rows; 0: chosen from the rows per expert) against the oracle's route: unpack (orc_dequant_w4_bf16, itself
    pinned by a brute-force check) then the bf16 grouped GEMM."""
    g = torch.Generator().manual_seed(E * n + k + (gs or 0))
    lod = _lod(counts)
    rows = int(lod[-1])
    group = gs or k
    packed = torch.randint(0, 256, (E, n, k // 2), generator=g, dtype=torch.uint8)
    scale = (torch.rand(E, n, k // group, generator=g) * 0.02 + 0.002).bfloat16()
    K = 2
    src_rows = (rows + K - 1) // K if gather else rows
    a = torch.randn(max(src_rows, 1), k, generator=g).bfloat16()
    row_src = torch.randperm(src_rows * K, generator=g)[:rows].int() if gather else None
    w_bits = co.dequant_w4_bf16(packed.numpy(), bits(scale), group)
    ref = co.grouped_gemm_bf16(bits(a), w_bits, lod, act=act, row_src=None if row_src is None else row_src.numpy(),
                               src_div=K if gather else 1)
    n_out = n // 2 if act else n
    dp = packed.cuda()
    dt = torch.empty_like(dp)
    L.check(L.lib.kmoe_tile_weights_i8(dp.data_ptr(), dt.data_ptr(), E, n, k // 2, L.stream()))
    da, ds, dl = a.cuda(), scale.cuda(), torch.from_numpy(lod).cuda()
    if frag16:  # the scales re-arranged per 16 channels, as the layer keeps them
        tiled = torch.empty_like(ds)
        L.check(L.lib.kmoe_tile_scales_w4(ds.data_ptr(), tiled.data_ptr(), E, n, k // group, L.stream()))
        want = ds.view(E, n // 16, 16, k // group).permute(0, 1, 3, 2).contiguous().view(E, n, k // group)
        assert torch.equal(tiled, want)
        ds = tiled
    dsrc = None if row_src is None else row_src.cuda()
    y = torch.zeros(rows, n_out, dtype=torch.bfloat16, device="cuda")
    args = L.GemmW4Args()
    args.scale_layout = L.KMOE_S_FRAG16 if frag16 else L.KMOE_S_ROWMAJOR
    args.a, args.lda, args.src_div = da.data_ptr(), k, K if gather else 1
    args.row_src = 0 if dsrc is None else dsrc.data_ptr()
    args.w, args.w_scale, args.group_size, args.lod = dt.data_ptr(), ds.data_ptr(), group, dl.data_ptr()
    args.E, args.n, args.k, args.rows = E, n, k, rows
    args.y, args.ldy, args.act, args.variant, args.w_layout = y.data_ptr(), n_out, act, variant, L.KMOE_W_TILED
    L.check(L.lib.kmoe_grouped_gemm_w4a16(args, L.stream()))
    torch.cuda.synchronize()
    assert rel_l2(y, from_bits(ref)) <= 2e-3   # the operands are the same bits: only summation order differs
    if variant >= 8:  # both kernels add the same products in the same order: the same bits
        y1 = torch.zeros_like(y)
        args.y, args.variant = y1.data_ptr(), 1
        L.check(L.lib.kmoe_grouped_gemm_w4a16(args, L.stream()))
        torch.cuda.synchronize()
        assert torch.equal(y, y1)
    # an independent torch statement of the unpacking and of one expert's product
    e = int(np.argmax(counts))
    r0, r1 = int(lod[e]), int(lod[e + 1])
    codes = torch.stack([packed[e] & 15, packed[e] >> 4], dim=-1).reshape(n, k).float() - 8.0
    w_e = (codes * scale[e].float().repeat_interleave(group, dim=1)).bfloat16().float()
    rows_e = a[(row_src[r0:r1] // K).long()] if gather else a[r0:r1]
    t = rows_e.float() @ w_e.T
    if act:
        t = tm.silu_and_mul(t.bfloat16()).float()
    assert rel_l2(y[r0:r1], t) <= REL_L2_BF16


def test_w4_scales_rearranged_in_place_and_back(L):
    """tile_w4_scales_ re-arranges group scales in place and marks the memory; the mark follows the memory, a view
    that cannot stand for it is refused, and rowmajor_w4_scales gives the checkpoint's values back."""
    from vllm_kunlun_amd import _plan
    g = torch.Generator().manual_seed(5)
    scale = torch.rand(3, 96, 7, generator=g).bfloat16().cuda()
    before = scale.clone()
    assert _plan.scale_layout(scale) == L.KMOE_S_ROWMAJOR
    assert _plan.tile_w4_scales_(scale) and _plan.tile_w4_scales_(scale)  # the second call finds the mark
    assert _plan.scale_layout(scale) == L.KMOE_S_FRAG16 and _plan.scale_layout(scale[1:]) == L.KMOE_S_FRAG16
    assert torch.equal(scale.view(3, 6, 7, 16), before.view(3, 6, 16, 7).transpose(2, 3))
    assert torch.equal(_plan.rowmajor_w4_scales(scale), before)
    with pytest.raises(ValueError):
        _plan.scale_layout(scale[:, :16])
    assert not _plan.tile_w4_scales_(torch.zeros(2, 24, 4, dtype=torch.bfloat16, device="cuda"))  # 24 channels


def test_grouped_gemm_w4a16_rejects_what_it_cannot_run(L):
    args = L.GemmW4Args()
    t = torch.zeros(64, dtype=torch.uint8, device="cuda")
    args.a = args.w = args.w_scale = args.lod = args.y = t.data_ptr()
    args.lda, args.ldy, args.src_div = 128, 64, 1
    args.E, args.n, args.k, args.rows, args.group_size = 1, 64, 128, 1, 128
    args.w_layout = L.KMOE_W_ROWMAJOR
    with pytest.raises(NotImplementedError):
        L.check(L.lib.kmoe_grouped_gemm_w4a16(args, L.stream()))
    args.w_layout, args.group_size = L.KMOE_W_TILED, 48
    with pytest.raises(ValueError):
        L.check(L.lib.kmoe_grouped_gemm_w4a16(args, L.stream()))
    args.group_size, args.k = 128, 192
    with pytest.raises(ValueError):
        L.check(L.lib.kmoe_grouped_gemm_w4a16(args, L.stream()))


@pytest.mark.parametrize("native", ["auto", "both", "only"])
@pytest.mark.parametrize("group_size,M", [(128, 24), (32, 5), (None, 24), (128, 700)])
def test_w4a16_layer_on_the_packed_weights(native, group_size, M):
    """The 4-bit method with shapes the packed-weight kernels take: kmoe_moe_forward with KMOE_FMT_W4A16
    (decode-sized batches on the streaming kernel, 700 tokens = 175 rows per expert on the tile kernel; with
    "both" that batch runs on the unpacked copy); against the C oracle on the unpacked weights."""
    from vllm_kunlun_amd.ops.fused_moe.layer import FusedMoE
    from vllm_kunlun_amd.quantization.compressed_tensors.compressed_tensors_moe import (
        KunlunCompressedTensorsWNA16MoEMethod)
    from types import SimpleNamespace
    E, H, I, K = 16, 256, 256, 4  # H == I: one scale per row is then one group size for both tensors
    wq = SimpleNamespace(num_bits=4, type="int", symmetric=True, dynamic=False,
                         strategy="group" if group_size else "channel", group_size=group_size)
    method = KunlunCompressedTensorsWNA16MoEMethod(wq, None, SimpleNamespace(experts_per_token=K), native=native)
    layer = FusedMoE(num_experts=E, top_k=K, hidden_size=H, intermediate_size=I, quant_method=method, device="cuda")
    g = torch.Generator().manual_seed(11)
    with torch.no_grad():
        for name, (n, k) in (("w13", (2 * I, H)), ("w2", (H, I))):
            getattr(layer, f"{name}_weight_packed").data = torch.randint(0, 256, (E, n, k // 2), generator=g,
                                                                         dtype=torch.uint8).cuda()
            getattr(layer, f"{name}_weight_scale").data = (torch.rand(E, n, k // (group_size or k), generator=g)
                                                           * 0.02 + 0.002).bfloat16().cuda()
    packed13, scale13 = layer.w13_weight_packed.data.cpu(), layer.w13_weight_scale.data.cpu()
    packed2, scale2 = layer.w2_weight_packed.data.cpu(), layer.w2_weight_scale.data.cpu()
    method.process_weights_after_loading(layer)
    assert layer.w4_native and hasattr(layer, "w13_weight_packed")
    assert hasattr(layer, "w13_weight") == (native == "both")
    gx = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(M, H, generator=gx, device="cuda").bfloat16()
    logits = torch.randn(M, E, generator=gx, device="cuda")
    out = layer(x, logits)
    torch.cuda.synchronize()
    w13 = co.dequant_w4_bf16(packed13.numpy(), bits(scale13), group_size or H)
    w2 = co.dequant_w4_bf16(packed2.numpy(), bits(scale2), group_size or I)
    ref = co.forward_bf16(bits(x), logits.cpu().numpy(), w13, w2, K)
    assert rel_l2(out, from_bits(ref)) <= REL_L2_BF16
    # the reference's entry point, argument for argument (compressed_tensors_moe.py:296-320): the same result, and
    # sigmoid scoring with a correction bias reaches the routing
    out2 = method.apply(layer, x, logits, K, True, use_grouped_topk=False, scoring_func="softmax")
    torch.cuda.synchronize()
    assert torch.equal(out2, out)
    bias = torch.randn(E, generator=torch.Generator().manual_seed(4)) * 0.1
    out3 = method.apply(layer, x, logits, K, True, scoring_func="sigmoid", e_score_correction_bias=bias.cuda())
    torch.cuda.synchronize()
    ref3 = co.forward_bf16(bits(x), logits.cpu().numpy(), w13, w2, K, scoring="sigmoid", bias=bias.numpy())
    assert rel_l2(out3, from_bits(ref3)) <= REL_L2_BF16
    # as rank 1 of 2 expert-parallel ranks: logits over 2 E experts, the layer's weights being experts E .. 2 E - 1
    ep = SimpleNamespace(experts_per_token=K, use_ep=True, ep_rank=1)
    method.moe, keep = ep, method.moe
    wide = torch.randn(M, 2 * E, generator=gx, device="cuda")
    out4 = method.apply(layer, x, wide, K, True)
    torch.cuda.synchronize()
    method.moe = keep
    ref4 = co.forward_bf16(bits(x), wide.cpu().numpy(), w13, w2, K, first_expert=E)
    assert rel_l2(out4, from_bits(ref4)) <= REL_L2_BF16
    with pytest.raises(NotImplementedError):
        method.apply(layer, x, logits, K, True, expert_map=torch.arange(E, device="cuda"))
    with pytest.raises(NotImplementedError):
        method.apply(layer, x, logits, K, True, activation="gelu")


@pytest.mark.parametrize("act", [None, "SWISH_GLU"])
@pytest.mark.parametrize("tiled", [False, True])
def test_moe_fc_op_block_scaled_fp8_and_packed_int4(act, tiled):
    """`_C::moe_fc` with scale_n / scale_k (block-scaled fp8 operands) and with use_pack_int4 (packed 4-bit
    weights): the operator's arguments reach the fp8 and the 4-bit grouped GEMM and give the oracle's result."""
    import vllm_kunlun_amd  # noqa: F401
    from vllm_kunlun_amd import _plan
    torch.manual_seed(77)
    E, n, k, counts = 3, 256, 384, [9, 0, 30]
    lod = _lod(counts)
    rows = int(lod[-1])
    dl = torch.from_numpy(lod).cuda()
    idx = torch.empty(0, dtype=torch.int32, device="cuda")
    n_out = n // 2 if act else n
    # fp8, 128 x 128 blocks
    x = (torch.randn(rows, k) * 2).bfloat16()
    xq, xs = tm.quant_fp8_group128(x)
    wq, ws = tm.quantize_weight_fp8_block128(torch.randn(E, n, k) * 0.02)
    ref = co.grouped_gemm_fp8(xq.view(torch.uint8).numpy(), xs.numpy(), wq.view(torch.uint8).numpy(), ws.numpy(), lod,
                              act=1 if act else 0)
    dw = wq.cuda()
    if tiled:
        assert _plan.tile_int8_weights_(dw)
    y = torch.zeros(rows, n_out, dtype=torch.bfloat16, device="cuda")
    torch.ops._C.moe_fc(xq.cuda(), dw, dl, idx, 1, y, act, xs.contiguous().cuda(), ws.contiguous().cuda(),
                        scale_n=128, scale_k=128)
    torch.cuda.synchronize()
    assert rel_l2(y, from_bits(ref)) <= 2e-3
    with pytest.raises(NotImplementedError):
        torch.ops._C.moe_fc(xq.cuda(), dw, dl, idx, 1, y, act, xs.cuda(), ws.cuda(), scale_n=64, scale_k=128)
    # packed 4-bit weights, groups of 128 along k; the kernel needs the packed bytes re-tiled
    g = torch.Generator().manual_seed(78)
    packed = torch.randint(0, 256, (E, n, k // 2), generator=g, dtype=torch.uint8)
    scale = (torch.rand(E, n, k // 128, generator=g) * 0.02 + 0.002).bfloat16()
    a = torch.randn(rows, k, generator=g).bfloat16()
    w_bits = co.dequant_w4_bf16(packed.numpy(), bits(scale), 128)
    ref4 = co.grouped_gemm_bf16(bits(a), w_bits, lod, act=1 if act else 0)
    dp = packed.cuda()
    y4 = torch.zeros(rows, n_out, dtype=torch.bfloat16, device="cuda")
    if not tiled:
        with pytest.raises(NotImplementedError):
            torch.ops._C.moe_fc(a.cuda(), dp, dl, idx, 1, y4, act, None, scale.cuda(), scale_k=128, use_pack_int4=True)
        return
    assert _plan.tile_int8_weights_(dp)
    torch.ops._C.moe_fc(a.cuda(), dp, dl, idx, 1, y4, act, None, scale.cuda(), scale_k=128, use_pack_int4=True)
    torch.cuda.synchronize()
    assert rel_l2(y4, from_bits(ref4)) <= 2e-3
