"""Pins the C oracle (oracle/moe_oracle.c) WITHOUT the reference: the reference
holds no test, fixture or golden vector for the MoE path and its arithmetic sits
in closed wheels, so each oracle function is tied down by what the mathematics
fixes — closed forms, exact integer arithmetic, brute force on tiny inputs,
invariants — and by independently written code: torch ops, the torch oracle, and
the DeepSeek-V3 / Qwen3-MoE router and expert modules of the `transformers`
library installed in the image. Each check is chosen so that a plausible slip
(dropped term, wrong sign or index, transposed operand, wrong tie-break) fails it.
"""
import itertools
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import bits, from_bits, rel_l2
from oracle import c_oracle as co
from oracle import torch_moe as tm


# ------------------------------------------------------------------ scalars
def test_exp_matches_libm_within_2ulp_and_is_monotone():
    xs = np.concatenate([np.linspace(-86, 86, 40001), np.linspace(-1, 1, 20001), [0.0, -0.0, 1e-30, -1e-30]])
    xs = xs.astype(np.float32)
    got = co.exp(xs).astype(np.float64)
    ref = np.exp(xs.astype(np.float64))
    ulp = np.spacing(ref.astype(np.float32)).astype(np.float64)
    assert np.max(np.abs(got - ref) / ulp) < 2.0
    order = np.argsort(xs, kind="stable")
    assert np.all(np.diff(got[order]) >= 0)
    assert co.exp(np.float32(0.0)) == 1.0


def test_exp_clamps_outside_range():
    assert co.exp(np.float32(-1000.0)) == co.exp(np.float32(-86.0)) > 0
    assert co.exp(np.float32(1000.0)) == co.exp(np.float32(86.0)) < np.inf


def test_sigmoid_and_silu_closed_forms():
    xs = np.linspace(-30, 30, 6001).astype(np.float32)
    s = co.sigmoid(xs).astype(np.float64)
    assert np.max(np.abs(s - 1 / (1 + np.exp(-xs.astype(np.float64))))) < 2e-7
    # symmetry sigma(x) + sigma(-x) = 1 and silu(x) - silu(-x) = x
    assert np.max(np.abs(s + co.sigmoid(-xs) - 1)) < 3e-7
    si = co.silu(xs).astype(np.float64)
    assert np.max(np.abs(si - co.silu(-xs) - xs)) < 4e-6
    assert co.silu(np.float32(0.0)) == 0.0
    assert abs(co.silu(np.float32(40.0)) - 40.0) < 1e-5 and abs(co.silu(np.float32(-40.0))) < 1e-10
    ref = F.silu(torch.from_numpy(xs).double()).numpy()
    assert np.max(np.abs(si - ref)) < 4e-6


# ------------------------------------------------------------------ routing
def _brute_topk(score, K, eligible=None):
    idx = [e for e in range(len(score)) if eligible is None or eligible[e]]
    idx.sort(key=lambda e: (-float(score[e]), e))
    return idx[:K]


@pytest.mark.parametrize("renorm", [False, True])
def test_softmax_topk_brute_force_and_closed_form(renorm):
    rng = np.random.default_rng(0)
    for E, K in [(4, 1), (8, 2), (16, 5), (70, 8), (130, 8)]:
        logits = rng.standard_normal((64, E)).astype(np.float32)
        logits[0, :3] = 1.25  # ties
        logits[1] = 0.0       # all tied: ids must be 0..K-1
        w, ids = co.softmax_topk(logits, K, renorm)
        p = torch.softmax(torch.from_numpy(logits).double(), -1).numpy()
        for m in range(logits.shape[0]):
            want = _brute_topk(logits[m], K)
            assert list(ids[m]) == want
            pw = p[m, want]
            if renorm:
                pw = pw / pw.sum()
            assert np.allclose(w[m], pw, rtol=2e-6, atol=1e-9)
        if renorm:
            assert np.allclose(w.sum(-1), 1.0, atol=1e-6)
        assert list(ids[1]) == list(range(K))


def test_softmax_topk_agrees_with_torch_and_transformers_router():
    from transformers.models.qwen3_moe.configuration_qwen3_moe import Qwen3MoeConfig
    from transformers.models.qwen3_moe.modeling_qwen3_moe import Qwen3MoeTopKRouter
    E, K, M = 128, 8, 512
    torch.manual_seed(1)
    logits = torch.randn(M, E)
    w, ids = co.softmax_topk(logits.numpy(), K, True)
    tw, tids = tm.softmax_topk(logits, K, True)
    assert np.array_equal(ids, tids.numpy())  # no exact ties in random normal data
    assert np.allclose(w, tw.numpy(), rtol=2e-6)
    cfg = Qwen3MoeConfig(hidden_size=E, num_experts=E, num_experts_per_tok=K, norm_topk_prob=True,
                         num_hidden_layers=1, vocab_size=8, intermediate_size=8, moe_intermediate_size=8)
    router = Qwen3MoeTopKRouter(cfg)
    with torch.no_grad():
        router.weight.copy_(torch.eye(E))  # logits = hidden_states
        _, rw, rids = router(logits)
    assert np.array_equal(ids, rids.numpy())
    assert np.allclose(w, rw.numpy(), rtol=2e-6)


def test_sigmoid_group_topk_brute_force():
    rng = np.random.default_rng(3)
    for E, K, ng, tg in [(8, 2, 4, 2), (16, 4, 4, 2), (16, 3, 1, 1), (12, 4, 3, 2), (16, 8, 8, 4)]:
        logits = rng.standard_normal((40, E)).astype(np.float32)
        bias = (rng.standard_normal(E) * 0.3).astype(np.float32)
        w, ids = co.sigmoid_group_topk_norm(logits, bias, K, ng, tg, 2.5)
        s = co.sigmoid(logits)
        c = (s + bias).astype(np.float32)
        gsz = E // ng
        for m in range(logits.shape[0]):
            if ng > 1:
                gscore = [np.float32(sum(sorted(c[m, g * gsz:(g + 1) * gsz], reverse=True)[:2])) for g in range(ng)]
                groups = _brute_topk(gscore, tg)
                elig = [e // gsz in groups for e in range(E)]
            else:
                elig = None
            want = _brute_topk(c[m], K, elig)
            assert list(ids[m]) == want
            sw = s[m, want].astype(np.float64)
            assert np.allclose(w[m], sw / sw.sum() * 2.5, rtol=3e-6)
            if ng > 1:
                assert len({e // gsz for e in ids[m]}) <= tg
        assert np.allclose(w.sum(-1), 2.5, rtol=1e-5)


def test_sigmoid_group_topk_special_case_reduces_to_plain_sigmoid_topk():
    rng = np.random.default_rng(4)
    logits = rng.standard_normal((50, 32)).astype(np.float32)
    w, ids = co.sigmoid_group_topk_norm(logits, None, 6, 1, 1, 1.0)
    for m in range(50):
        assert list(ids[m]) == _brute_topk(logits[m], 6)  # sigmoid is monotone, bias 0
    w0, ids0 = co.sigmoid_group_topk_norm(logits, np.zeros(32, np.float32), 6, 1, 1, 1.0)
    assert np.array_equal(ids, ids0) and np.array_equal(w, w0)


def test_sigmoid_group_topk_agrees_with_transformers_deepseek_v3_router():
    from transformers.models.deepseek_v3.configuration_deepseek_v3 import DeepseekV3Config
    from transformers.models.deepseek_v3.modeling_deepseek_v3 import DeepseekV3TopkRouter
    E, K, ng, tg, M = 256, 8, 8, 4, 256
    cfg = DeepseekV3Config(hidden_size=E, n_routed_experts=E, num_experts_per_tok=K, n_group=ng, topk_group=tg,
                           routed_scaling_factor=2.5, norm_topk_prob=True, num_hidden_layers=1, intermediate_size=8,
                           moe_intermediate_size=8, vocab_size=8)
    router = DeepseekV3TopkRouter(cfg)
    torch.manual_seed(5)
    logits = torch.randn(M, E)
    bias = torch.randn(E) * 0.01
    with torch.no_grad():
        router.weight.copy_(torch.eye(E))
        router.e_score_correction_bias.copy_(bias)
        _, rw, rids = router(logits)
    w, ids = co.sigmoid_group_topk_norm(logits.numpy(), bias.numpy(), K, ng, tg, 2.5)
    # the library returns the K experts unsorted: compare as sets, weights by expert
    for m in range(M):
        mine = dict(zip(ids[m].tolist(), w[m].tolist()))
        theirs = dict(zip(rids[m].tolist(), rw[m].tolist()))
        assert set(mine) == set(theirs)
        for e in mine:
            assert math.isclose(mine[e], theirs[e], rel_tol=3e-6)
    tw, tids = tm.sigmoid_group_topk_norm(logits, bias, K, ng, tg, 2.5)
    assert np.array_equal(np.sort(ids, -1), np.sort(tids.numpy(), -1))


# -------------------------------------------------------------------- align
@pytest.mark.parametrize("P,E", [(0, 4), (1, 4), (100, 7), (4096, 128), (5000, 1024)])
def test_align_closed_form(P, E):
    rng = np.random.default_rng(P + E)
    ids = rng.integers(0, E, P).astype(np.int32)
    moe_index, sorted_src, expert_m, lod = co.align(ids, E)
    order = np.argsort(ids, kind="stable")
    assert np.array_equal(sorted_src, order)
    assert np.array_equal(expert_m, np.bincount(ids, minlength=E))
    assert np.array_equal(lod, np.concatenate([[0], np.cumsum(expert_m)]))
    inv = np.empty(P, np.int64)
    inv[order] = np.arange(P)
    assert np.array_equal(moe_index, inv)
    t_mi, t_src, t_em, t_lod = tm.align(torch.from_numpy(ids), E)
    assert np.array_equal(moe_index, t_mi.numpy()) and np.array_equal(lod, t_lod.numpy())


def test_align_properties_hypothesis():
    from hypothesis import given, settings
    from hypothesis import strategies as st

    @settings(max_examples=60, deadline=None)
    @given(st.integers(1, 40).flatmap(lambda E: st.tuples(st.just(E), st.lists(st.integers(0, E - 1), max_size=300))))
    def prop(args):
        E, lst = args
        ids = np.array(lst, dtype=np.int32)
        P = ids.size
        moe_index, sorted_src, expert_m, lod = co.align(ids, E)
        assert lod[0] == 0 and lod[E] == P and np.all(np.diff(lod) == expert_m)
        assert sorted(moe_index.tolist()) == list(range(P))          # a permutation
        assert np.all(np.diff(ids[sorted_src]) >= 0) if P else True    # experts non-decreasing
        for e in range(E):                                             # stable inside an expert
            seg = sorted_src[lod[e]:lod[e + 1]]
            assert np.all(np.diff(seg) > 0) and np.all(ids[seg] == e)
        assert np.array_equal(sorted_src[moe_index], np.arange(P))

    prop()


def test_block_statistic_sums_to_histogram():
    ids = np.random.default_rng(0).integers(0, 50, 1234).astype(np.int32)
    bs = co.block_statistic(ids, 50, 12)
    assert np.array_equal(bs.sum(0), np.bincount(ids, minlength=50))
    per = -(-1234 // 12)
    assert np.array_equal(bs[3], np.bincount(ids[3 * per:4 * per], minlength=50))


# -------------------------------------------------------------------- quant
def test_quant_i8_rows_closed_form_and_invariants():
    torch.manual_seed(0)
    x = (torch.randn(64, 1000) * 3).bfloat16()
    x[0] = 0
    x[1] = -2.0
    q, mx = co.quant_i8_rows(bits(x))
    xf = x.float().numpy()
    assert np.array_equal(mx, np.abs(xf).max(-1))
    assert np.all(q[0] == 0) and mx[0] == 0
    assert np.all(q[1] == -127)
    with np.errstate(divide="ignore", invalid="ignore"):
        inv = np.where(mx > 0, np.float32(127.0) / mx, np.float32(0))[:, None].astype(np.float32)
    want = np.clip(np.rint(xf * inv), -127, 127).astype(np.int8)  # np.rint = half-to-even
    assert np.array_equal(q, want)
    assert np.abs(q).max() <= 127
    am = np.abs(xf).argmax(-1)
    assert np.all(np.abs(q[np.arange(64), am])[mx > 0] == 127)       # the max element maps to +-127
    err = np.abs(xf - q.astype(np.float32) * mx[:, None] / 127)
    assert np.all(err <= mx[:, None] / 254 * 1.0001 + 1e-12)         # half a step
    tq, tmx = tm.quant_i8_rows(x)
    # torch evaluates 127/max with its own vectorised division: codes may differ by one
    # at exact .5 boundaries, nowhere else
    dq = np.abs(q.astype(np.int32) - tq.numpy().astype(np.int32))
    assert dq.max() <= 1 and (dq != 0).mean() < 1e-3 and np.array_equal(mx, tmx.numpy().ravel())


def test_quant_i8_rounds_half_to_even():
    # max = 127 makes the scale exactly 1: values k + 0.5 must go to the even neighbour
    vals = torch.tensor([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5]]).bfloat16()
    q, mx = co.quant_i8_rows(bits(vals))
    assert mx[0] == 127.0
    assert q[0].tolist() == [127, 0, 2, 2, 0, -2, -2, 4]


def test_e4m3fn_encoder_matches_torch_cast():
    # every representable value round-trips; random values match torch's RNE cast
    codes = np.arange(0, 0x7F, dtype=np.uint8)
    vals = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    for c, v in zip(codes, vals):
        assert co.lib().orc_f32_to_e4m3fn(float(v)) == c
        assert co.lib().orc_e4m3fn_to_f32(int(c)) == v
    rng = np.random.default_rng(0)
    xs = np.concatenate([rng.standard_normal(4000) * 100, rng.standard_normal(4000) * 0.01,
                         (vals[:-1] + vals[1:]) / 2, [448.0, 449.0, 1e9, -1e9, 2.0 ** -10, 2.0 ** -9 * 1.5]])
    xs = xs.astype(np.float32)
    want = torch.from_numpy(xs).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = np.array([co.lib().orc_f32_to_e4m3fn(float(v)) for v in xs], dtype=np.uint8)
    nz = (want & 0x7F) != 0  # torch keeps the sign of values that round to zero; so do we
    assert np.array_equal(got[nz], want[nz])
    assert np.all((got[~nz] & 0x7F) == 0)


def test_quant_fp8_group128_closed_form():
    torch.manual_seed(1)
    x = (torch.randn(9, 384) * 5).bfloat16()
    x[0, :128] = 0
    q, s = co.quant_fp8_group128(bits(x))
    tq, ts = tm.quant_fp8_group128(x)
    assert np.array_equal(s, ts.numpy())
    assert np.array_equal(s, np.abs(x.float().numpy().reshape(9, 3, 128)).max(-1) / np.float32(448.0))
    a, b = q, tq.view(torch.uint8).numpy()
    nz = (b & 0x7F) != 0
    assert np.array_equal(a[nz], b[nz]) and np.all((a[~nz] & 0x7F) == 0)
    assert np.all(q[0, :128] == 0) and s[0, 0] == 0


# --------------------------------------------------------------- grouped GEMM
def test_grouped_gemm_accumulators_are_exact_integers():
    rng = np.random.default_rng(0)
    E, n, k = 5, 48, 320
    counts = np.array([3, 0, 11, 1, 6])
    lod = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    rows = int(lod[-1])
    a = rng.integers(-127, 128, (rows, k), dtype=np.int8)
    w = rng.integers(-127, 128, (E, n, k), dtype=np.int8)
    a_max = (rng.random(rows) + 0.5).astype(np.float32)
    w_max = (rng.random((E, n)) + 0.5).astype(np.float32)
    y, acc = co.grouped_gemm_i8(a, a_max, w, w_max, lod, want_acc=True)
    for e in range(E):
        r0, r1 = lod[e], lod[e + 1]
        want = a[r0:r1].astype(np.int64) @ w[e].astype(np.int64).T          # textbook, int64
        assert np.array_equal(acc[r0:r1], want)
        assert np.array_equal(acc[r0:r1], tm._int8_mm(torch.from_numpy(a[r0:r1]), torch.from_numpy(w[e])).numpy())
        deq = (want.astype(np.float32) * (a_max[r0:r1, None] / np.float32(127))) * (w_max[e][None] / np.float32(127))
        assert np.array_equal(y[r0:r1], co.f32_to_bf16_bits(deq))            # one fixed f32 order, bf16 RNE
    # transposing the weight operand, or using the wrong expert's block, must fail the check above:
    assert not np.array_equal(acc[lod[2]:lod[3]], a[lod[2]:lod[3]].astype(np.int64) @ w[0].astype(np.int64).T)


def test_grouped_gemm_row_gather_and_swiglu():
    rng = np.random.default_rng(1)
    E, n, k, K = 3, 64, 128, 2
    tokens = 10
    a = rng.integers(-127, 128, (tokens, k), dtype=np.int8)
    a_max = (rng.random(tokens) + 0.5).astype(np.float32)
    w = rng.integers(-127, 128, (E, n, k), dtype=np.int8)
    w_max = (rng.random((E, n)) * 0.05 + 0.01).astype(np.float32)
    ids = rng.integers(0, E, tokens * K).astype(np.int32)
    _, src, _, lod = co.align(ids, E)
    y_gather, _ = co.grouped_gemm_i8(a, a_max, w, w_max, lod, row_src=src, src_div=K)
    y_expanded, _ = co.grouped_gemm_i8(a[src // K], a_max[src // K], w, w_max, lod)
    assert np.array_equal(y_gather, y_expanded)           # gather == the reference's expanded copy
    fused, _ = co.grouped_gemm_i8(a, a_max, w, w_max, lod, act=1, row_src=src, src_div=K)
    assert np.array_equal(fused, co.silu_and_mul(y_gather))  # fused act == act on the stored bf16 tensor


def test_bf16_round_trip_helpers():
    x = torch.randn(1000).float()
    assert np.array_equal(co.f32_to_bf16_bits(x.numpy()), bits(x.bfloat16()))
    assert np.array_equal(co.bf16_bits_to_f32(bits(x.bfloat16())), x.bfloat16().float().numpy())


def test_silu_and_mul_against_torch():
    torch.manual_seed(2)
    y = (torch.randn(33, 96) * 3).bfloat16()
    got = from_bits(co.silu_and_mul(bits(y))).float()
    want = tm.silu_and_mul(y).float()
    assert (got - want).abs().max() <= 2 ** -7 * want.abs().max()   # at most 1 bf16 ulp apart
    assert (got == want).float().mean() > 0.98
    # gate is the FIRST half: swapping halves must change the result
    swapped = from_bits(co.silu_and_mul(bits(torch.cat([y[:, 48:], y[:, :48]], 1)))).float()
    assert not torch.equal(swapped, got)


def test_combine_closed_form():
    torch.manual_seed(3)
    M, K, H = 20, 4, 64
    x = torch.randn(M * K, H).bfloat16()
    w = torch.rand(M, K)
    perm = torch.randperm(M * K).int()
    got = from_bits(co.combine(bits(x), perm.numpy(), w.numpy())).double()
    want = (x.double()[perm.long()].view(M, K, H) * w.double().unsqueeze(-1)).sum(1)
    assert (got - want).abs().max() <= 2 ** -8 * want.abs().max() + 1e-6
    # equal weights: permuting the K slots of a token only changes f32 summation order
    w1 = torch.full((M, K), 0.25)
    a = from_bits(co.combine(bits(x), perm.numpy(), w1.numpy())).float()
    b = from_bits(co.combine(bits(x), perm.view(M, K).flip(1).contiguous().numpy(), w1.numpy())).float()
    assert (a - b).abs().max() <= 2 ** -7 * a.abs().max()
    # caller epilogue: bf16(out*scale) + addend
    add = torch.randn(M, H).bfloat16()
    e = from_bits(co.combine(bits(x), perm.numpy(), w.numpy(), None, 2.5, bits(add)))
    base = from_bits(co.combine(bits(x), perm.numpy(), w.numpy()))
    assert torch.equal(e, (base * 2.5) + add)


# ------------------------------------------------------------- whole layer
def _layer_inputs(M, H, E, K, I, seed, shared_I=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, H, generator=g).bfloat16()
    logits = torch.randn(M, E, generator=g)
    w13, s13 = tm.quantize_weight_per_channel(torch.randn(E, 2 * I, H, generator=g) * 0.02)
    w2, s2 = tm.quantize_weight_per_channel(torch.randn(E, H, I, generator=g) * 0.02)
    shared = None
    if shared_I:
        a, sa = tm.quantize_weight_per_channel(torch.randn(2 * shared_I, H, generator=g) * 0.02)
        b, sb = tm.quantize_weight_per_channel(torch.randn(H, shared_I, generator=g) * 0.02)
        shared = (a, (sa * 127).reshape(-1), b, (sb * 127).reshape(-1))
    return x, logits, w13, s13 * 127, w2, s2 * 127, shared


def test_layer_c_oracle_vs_torch_expert_loop():
    """Two independently written restatements of the reference layer agree within the
    north-star tolerance; routing ids agree exactly."""
    M, H, E, K, I = 96, 256, 16, 4, 128
    x, logits, w13, m13, w2, m2, shared = _layer_inputs(M, H, E, K, I, 0, shared_I=64)
    bias = torch.randn(E) * 0.01
    for kw in (dict(scoring="softmax"), dict(scoring="sigmoid", n_group=4, topk_group=2, routed_scale=2.5, bias=bias)):
        ref = tm.w8a8_moe(x, logits, w13, m13, w2, m2, K, shared=shared, out_scale=1.0,
                          **{k: v for k, v in kw.items()})
        np_kw = dict(kw)
        if "bias" in np_kw:
            np_kw["bias"] = bias.numpy()
        out, inter = co.forward_w8a8(bits(x), logits.numpy(), w13.numpy(), m13.numpy(), w2.numpy(), m2.numpy(), K,
                                     shared=tuple(t.numpy() for t in shared), intermediates=True, **np_kw)
        assert rel_l2(from_bits(out), ref) <= 1e-2
        tw, tids = tm.route(logits, K, kw["scoring"], True, kw.get("n_group", 1), kw.get("topk_group", 1),
                            kw.get("routed_scale", 1.0), kw.get("bias"))
        assert np.array_equal(np.sort(inter["topk_ids"], -1), np.sort(tids.numpy(), -1))


def test_layer_against_transformers_deepseek_experts_on_dequantised_weights():
    """Independent end-to-end anchor: the library's float expert loop on the
    DEQUANTISED weights; the W8A8 layer may differ only by quantisation noise."""
    from transformers.models.deepseek_v3.configuration_deepseek_v3 import DeepseekV3Config
    from transformers.models.deepseek_v3.modeling_deepseek_v3 import DeepseekV3Experts
    M, H, E, K, I = 64, 256, 8, 2, 128
    x, logits, w13, m13, w2, m2, _ = _layer_inputs(M, H, E, K, I, 7)
    cfg = DeepseekV3Config(hidden_size=H, n_routed_experts=E, num_local_experts=E, moe_intermediate_size=I,
                           num_experts_per_tok=K, num_hidden_layers=1, intermediate_size=8, vocab_size=8)
    experts = DeepseekV3Experts(cfg)
    with torch.no_grad():
        experts.gate_up_proj.copy_(w13.float() * (m13 / 127))
        experts.down_proj.copy_(w2.float() * (m2 / 127))
        w, ids = co.softmax_topk(logits.numpy(), K, True)
        ref = experts(x.float(), torch.from_numpy(ids).long(), torch.from_numpy(w))
    out = co.forward_w8a8(bits(x), logits.numpy(), w13.numpy(), m13.numpy(), w2.numpy(), m2.numpy(), K)
    assert rel_l2(from_bits(out), ref) <= 3e-2   # int8 activation quantisation noise only
    # a swapped gate/up or a transposed down projection is far outside this band
    with torch.no_grad():
        experts.gate_up_proj.copy_(torch.cat([experts.gate_up_proj[:, I:], experts.gate_up_proj[:, :I]], 1))
        bad = experts(x.float(), torch.from_numpy(ids).long(), torch.from_numpy(w))
    assert rel_l2(from_bits(out), bad) > 0.3


def test_process_weights_scale_times_127_is_the_max_convention():
    """scale -> max: dequantising with max/127 must reproduce scale (reference:
    compressed_tensors_moe.py:116-120, scale_mm.py:43-50)."""
    w = torch.randn(3, 16, 32) * 0.02
    q, s = tm.quantize_weight_per_channel(w)
    mx = s * 127.0
    assert torch.allclose(mx, w.abs().amax(-1, keepdim=True), rtol=1e-6)
    assert (q.float() * (mx / 127.0) - w).abs().max() <= (s.max() / 2) * 1.001


def test_bf16_expert_loop_matches_float_math():
    """The unquantized torch loop (config 1: 32 tokens, hidden 512, 8 experts, top-2, I=256)."""
    g = torch.Generator().manual_seed(0)
    M, H, E, K, I = 32, 512, 8, 2, 256
    x = torch.randn(M, H, generator=g).bfloat16()
    logits = torch.randn(M, E, generator=g)
    w13 = (torch.randn(E, 2 * I, H, generator=g) * 0.02).bfloat16()
    w2 = (torch.randn(E, H, I, generator=g) * 0.02).bfloat16()
    out = tm.bf16_moe(x, logits, w13, w2, K, True)
    p = torch.softmax(logits.double(), -1)
    tw, ti = p.topk(K, -1)
    tw = tw / tw.sum(-1, keepdim=True)
    ref = torch.zeros(M, H, dtype=torch.double)
    for m in range(M):
        for k in range(K):
            e = ti[m, k]
            h = x[m].double() @ w13[e].double().T
            ref[m] += tw[m, k] * ((F.silu(h[:I]) * h[I:]) @ w2[e].double().T)
    assert rel_l2(out, ref) <= 1e-2


def test_router_gemm_against_f64_matmul():
    """logits = x . w^T: exact products, double sum, one rounding; a transposed operand, a wrong
    stride or a dropped k would show against torch's f64 matmul; abs_sum is sum |x*w|."""
    torch.manual_seed(11)
    for M, H, E in ((1, 32, 1), (5, 96, 7), (33, 256, 130)):
        x = torch.randn(M, H).bfloat16()
        w = (torch.randn(E, H) * 0.05).bfloat16()
        got, abs_sum = co.router_gemm(bits(x), bits(w))
        ref = x.double() @ w.double().T
        assert np.array_equal(got, ref.float().numpy())
        assert np.allclose(abs_sum, (x.double().abs() @ w.double().abs().T).numpy(), rtol=1e-6)


def test_swigluoai_matches_the_reference_definition_and_its_clamps():
    """The C oracle's gpt-oss activation against the reference's own torch definition
    (restated in oracle/torch_moe.py from ops/_custom_ops.py:728-742) evaluated in f32, and the
    closed forms at the clamps: a dropped `+1`, a swapped gate/up or a missing clamp fails."""
    torch.manual_seed(3)
    y = (torch.randn(64, 96) * 4).bfloat16()
    y[0, :8] = torch.tensor([9.0, 0.5, -3.0, 9.0, 0.0, 2.0, 1.0, -9.0]).bfloat16()
    got = from_bits(co.swigluoai_and_mul(bits(y))).float()
    ref = tm.swigluoai_and_mul(y.float())
    assert rel_l2(got, ref) < 3e-3
    assert torch.allclose(got, ref, rtol=2 ** -7, atol=1e-6)
    a, lim = 1.702, 7.0
    sig = lambda v: 1.0 / (1.0 + math.exp(-v))  # noqa: E731
    want = [(0.5 + 1) * lim * sig(a * lim),      # gate 9 -> limit
            (lim + 1) * -3.0 * sig(a * -3.0),    # up 9 -> limit
            0.0,                                  # gate 0
            (-lim + 1) * 1.0 * sig(a * 1.0)]      # up -9 -> -limit
    assert np.allclose(got[0, :4].numpy(), want, rtol=2 ** -7)


def test_expert_bias_branch_against_the_reference_loop():
    """C oracle forward with expert biases vs the reference's gpt-oss torch loop
    (ops/_kunlun_ops.py:433-468, restated in oracle/torch_moe.py)."""
    torch.manual_seed(8)
    M, H, E, K, I = 24, 64, 6, 2, 32
    x = torch.randn(M, H).bfloat16()
    logits = torch.randn(M, E)
    w13 = (torch.randn(E, 2 * I, H) * 0.1).bfloat16()
    w2 = (torch.randn(E, H, I) * 0.1).bfloat16()
    b13 = (torch.randn(E, 2 * I) * 0.2).bfloat16()
    b2 = (torch.randn(E, H) * 0.2).bfloat16()
    got = from_bits(co.forward_bf16(bits(x), logits.numpy(), bits(w13), bits(w2), K, w13_bias=bits(b13),
                                    w2_bias=bits(b2)))
    ref = tm.bf16_moe_bias(x, logits, w13, w2, b13, b2, K)
    assert rel_l2(got, ref) <= 1e-2
    no_b2 = from_bits(co.forward_bf16(bits(x), logits.numpy(), bits(w13), bits(w2), K, w13_bias=bits(b13)))
    assert rel_l2(no_b2, tm.bf16_moe_bias(x, logits, w13, w2, b13, None, K)) <= 1e-2
    assert rel_l2(no_b2, ref) > 5e-2   # the down bias matters


def test_dequant_w4_against_the_reference_expression():
    """Low nibble first, code - 8, times the scale (quantization/kernels/quant_ops.py:71-86, with
    contiguous groups): checked against that expression written with torch ops."""
    torch.manual_seed(5)
    for rows, k, gs in ((3, 32, 32), (4, 64, 16), (2, 256, 128)):
        packed = torch.randint(0, 256, (rows, k // 2), dtype=torch.uint8)
        scale = (torch.rand(rows, k // gs) * 0.1 + 0.01).bfloat16()
        got = from_bits(co.dequant_w4_bf16(packed.numpy(), bits(scale), gs))
        codes = torch.stack((packed & 0xF, (packed >> 4) & 0xF), dim=-1).reshape(rows, k).float() - 8.0
        ref = (codes * scale.float().repeat_interleave(gs, dim=1)).bfloat16()
        assert torch.equal(got, ref)
    one = co.dequant_w4_bf16(np.array([[0x1F] * 8], np.uint8), bits(torch.tensor([[2.0]]).bfloat16()), 16)
    assert from_bits(one).tolist()[0][:2] == [14.0, -14.0]   # 0xF - 8 = 7 first (low nibble), 0x1 - 8 = -7 second


def test_dequant_w4_half_is_the_reference_statement_in_float16():
    """The float16 mode against dequant_int4_native written out with torch's own float16 arithmetic
    (quantization/kernels/quant_ops.py:71-86: stack the nibbles, .to(float16) - 8.0, *= the scale; contiguous
    groups): bit for bit, scales down to subnormal products included."""
    torch.manual_seed(6)
    for rows, k, gs, lo in ((3, 32, 32, 0.01), (4, 64, 16, 0.01), (2, 256, 128, 0.01), (5, 64, 32, 1e-6)):
        packed = torch.randint(0, 256, (rows, k // 2), dtype=torch.uint8)
        scale = (torch.rand(rows, k // gs) * lo * 10 + lo).half()
        got = co.dequant_w4_bf16(packed.numpy(), scale.view(torch.int16).numpy().view(np.uint16), gs, f16=True)
        w = torch.stack((packed & 0xF, (packed >> 4) & 0xF), dim=-1).reshape(rows, k).contiguous().to(torch.float16) - 8.0
        w *= scale.repeat_interleave(gs, dim=1)
        assert np.array_equal(got, w.view(torch.int16).numpy().view(np.uint16))
    # the mode is per call: the next bf16 call is unaffected
    one = co.dequant_w4_bf16(np.array([[0x1F] * 8], np.uint8), bits(torch.tensor([[2.0]]).bfloat16()), 16)
    assert from_bits(one).tolist()[0][:2] == [14.0, -14.0]


# ------------------------------------------- bf16 and fp8 grouped GEMMs, and the layers built on them
def _fp8_codes(t: torch.Tensor) -> np.ndarray:
    """float tensor -> e4m3fn code bytes (torch's cast rounds to nearest even; values clamped to +-448 first,
    the cast itself does not saturate)."""
    return t.clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8).numpy()


def _fp8_values(codes: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(codes).view(torch.float8_e4m3fn).double()


def test_grouped_gemm_bf16_against_f64_matmul_and_its_gather():
    """y = bf16(a . w[e]^T) per expert: an f64 matmul of the same bf16 values differs by f32 summation and
    one rounding only (rel-L2 of a few 1e-3, every element within 2 bf16 steps of the f64 result's scale);
    the wrong expert's weights, a transposed operand or a dropped k is far outside. Gather == expanded copy,
    fused SiLU-mul == silu_and_mul of the stored result, bit for bit."""
    g = torch.Generator().manual_seed(21)
    E, n, k, K, tokens = 4, 96, 160, 2, 9
    a = torch.randn(tokens, k, generator=g).bfloat16()
    w = (torch.randn(E, n, k, generator=g) * 0.05).bfloat16()
    ids = torch.randint(0, E, (tokens * K,), generator=g).int().numpy()
    ids[ids == 2] = 3                                   # expert 2 stays empty
    _, src, _, lod = co.align(ids, E)
    y = co.grouped_gemm_bf16(bits(a), bits(w), lod, row_src=src, src_div=K)
    rows = a[torch.from_numpy(src // K).long()]
    assert np.array_equal(y, co.grouped_gemm_bf16(bits(rows), bits(w), lod))          # gather == expanded copy
    got = from_bits(y).double()
    for e in range(E):
        r0, r1 = int(lod[e]), int(lod[e + 1])
        if r1 == r0:
            continue
        ref = rows[r0:r1].double() @ w[e].double().T
        assert rel_l2(got[r0:r1], ref) <= 4e-3
        assert float((got[r0:r1] - ref).abs().max()) <= ref.abs().max() * 2 ** -7
        other = rows[r0:r1].double() @ w[(e + 1) % E].double().T
        assert rel_l2(got[r0:r1], other) > 0.5                                         # the wrong expert's block
    fused = co.grouped_gemm_bf16(bits(a), bits(w), lod, act=1, row_src=src, src_div=K)
    assert np.array_equal(fused, co.silu_and_mul(y))


def test_grouped_gemm_unquantized_half_against_f64_matmul():
    """The unquantized GEMM in its float16 mode: the same checks as for bf16, with numpy's float16 as the
    independent statement of the operand decoding and the result rounding (the f64 product rounded to half
    differs from the f32-summed one by at most one half step, rarely); fused SiLU-mul == the half SiLU-mul
    of the stored result, bit for bit."""
    rng = np.random.default_rng(23)
    E, n, k, K, tokens = 3, 64, 96, 2, 8
    a = rng.standard_normal((tokens, k)).astype(np.float16)
    w = (rng.standard_normal((E, n, k)) * 0.05).astype(np.float16)
    ids = rng.integers(0, E, tokens * K).astype(np.int32)
    ids[ids == 1] = 2                                   # expert 1 stays empty
    _, src, _, lod = co.align(ids, E)
    y = co.grouped_gemm_bf16(a.view(np.uint16), w.view(np.uint16), lod, row_src=src, src_div=K, f16=True)
    rows = a[src // K]
    assert np.array_equal(y, co.grouped_gemm_bf16(rows.view(np.uint16), w.view(np.uint16), lod, f16=True))
    got = y.view(np.float16).astype(np.float64)
    for e in range(E):
        r0, r1 = int(lod[e]), int(lod[e + 1])
        if r1 == r0:
            continue
        ref = rows[r0:r1].astype(np.float64) @ w[e].astype(np.float64).T
        ref_h = ref.astype(np.float16).astype(np.float64)
        assert np.abs(got[r0:r1] - ref_h).max() <= np.spacing(np.abs(ref_h).max().astype(np.float16)).astype(np.float64)
        assert np.mean(got[r0:r1] == ref_h) > 0.98
        assert np.linalg.norm(got[r0:r1] - ref) / np.linalg.norm(ref) <= 5e-4   # bf16 would sit at 3e-3
    fused = co.grouped_gemm_bf16(a.view(np.uint16), w.view(np.uint16), lod, act=1, row_src=src, src_div=K, f16=True)
    assert np.array_equal(fused, co.silu_and_mul(y, f16=True))
    # and the mode does not leak into the next bf16 call
    ab, wb = bits(torch.from_numpy(a.astype(np.float32)).bfloat16()), bits(torch.from_numpy(w.astype(np.float32)).bfloat16())
    yb = co.grouped_gemm_bf16(ab, wb, lod, row_src=src, src_div=K)
    assert rel_l2(from_bits(yb)[: int(lod[1])], torch.from_numpy(got[: int(lod[1])])) <= 1e-2


def test_grouped_gemm_fp8_against_f64_block_scaled_product():
    """y[r,c] = sum over 128-wide K blocks of (q_a . q_w) * s_a[r,kb] * s_w[e, c/128, kb]. Checked against
    the same expression in f64 on torch's decoding of the codes. The scales differ per (row, block) and per
    (channel block, K block) by factors of up to 8, so that swapping the two scale indices, taking one
    scale for all blocks or dropping a block is far outside the tolerance (shown below for each)."""
    g = torch.Generator().manual_seed(22)
    E, n, k, K, tokens = 3, 256, 384, 2, 7
    kb, nb = k // 128, n // 128
    aq = _fp8_codes(torch.randn(tokens, k, generator=g) * 100)
    wq = _fp8_codes(torch.randn(E, n, k, generator=g) * 100)
    a_s = (2.0 ** torch.randint(-3, 1, (tokens, kb), generator=g).float()).numpy() * 1e-2
    w_s = (2.0 ** torch.randint(-3, 1, (E, nb, kb), generator=g).float()).numpy() * 1e-3
    ids = torch.randint(0, E, (tokens * K,), generator=g).int().numpy()
    _, src, _, lod = co.align(ids, E)
    y = co.grouped_gemm_fp8(aq, a_s, wq, w_s, lod, row_src=src, src_div=K)
    tok = src // K
    assert np.array_equal(y, co.grouped_gemm_fp8(aq[tok], a_s[tok], wq, w_s, lod))      # gather == expanded copy
    got = from_bits(y).double()
    af = _fp8_values(aq)[torch.from_numpy(tok).long()].view(-1, kb, 128)
    sa = torch.from_numpy(a_s).double()[torch.from_numpy(tok).long()]

    def product(e, r0, r1, sa_rows, sw):
        wf = _fp8_values(wq[e]).view(n, kb, 128)
        part = torch.einsum("rbk,nbk->rnb", af[r0:r1], wf)                             # [rows, n, kb], exact in f64
        return (part * sa_rows[:, None, :] * sw.repeat_interleave(128, dim=0)[None]).sum(-1)

    for e in range(E):
        r0, r1 = int(lod[e]), int(lod[e + 1])
        if r1 == r0:
            continue
        sw = torch.from_numpy(w_s[e]).double()
        ref = product(e, r0, r1, sa[r0:r1], sw)
        assert rel_l2(got[r0:r1], ref) <= 4e-3
        assert float((got[r0:r1] - ref).abs().max()) <= ref.abs().max() * 2 ** -7
        # plausible slips, each far outside: K-block order of either scale reversed, one scale for all blocks,
        # the last K block dropped, the channel-block index of the weight scale swapped
        assert rel_l2(got[r0:r1], product(e, r0, r1, sa[r0:r1].flip(1), sw)) > 0.1
        assert rel_l2(got[r0:r1], product(e, r0, r1, sa[r0:r1], sw.flip(1))) > 0.1
        assert rel_l2(got[r0:r1], product(e, r0, r1, sa[r0:r1, :1].expand(-1, kb), sw)) > 0.1
        assert rel_l2(got[r0:r1], product(e, r0, r1, sa[r0:r1], sw.flip(0))) > 0.1
        dropped = sa[r0:r1].clone()
        dropped[:, -1] = 0
        assert rel_l2(got[r0:r1], product(e, r0, r1, dropped, sw)) > 0.1
    # act=1 is silu_and_mul of the stored act=0 result (gate = first half of the channels, up = second)
    fused = co.grouped_gemm_fp8(aq, a_s, wq, w_s, lod, act=1, row_src=src, src_div=K)
    assert np.array_equal(fused, co.silu_and_mul(y))


def test_forward_bf16_without_biases_against_a_per_expert_loop():
    """co.forward_bf16 (routing -> sort -> gate_up + SiLU-mul -> down -> combine) against a plain torch loop
    in f64 over the same bf16 weights, softmax and sigmoid-grouped routing."""
    g = torch.Generator().manual_seed(23)
    M, H, E, K, I = 19, 128, 8, 3, 64
    x = torch.randn(M, H, generator=g).bfloat16()
    logits = torch.randn(M, E, generator=g)
    w13 = (torch.randn(E, 2 * I, H, generator=g) * 0.05).bfloat16()
    w2 = (torch.randn(E, H, I, generator=g) * 0.05).bfloat16()
    bias = torch.randn(E, generator=g) * 0.01
    for scoring, n_group, topk_group, scale in (("softmax", 1, 1, 1.0), ("sigmoid", 4, 2, 2.5)):
        out = co.forward_bf16(bits(x), logits.numpy(), bits(w13), bits(w2), K, scoring, True, n_group, topk_group,
                              scale, bias.numpy() if scoring == "sigmoid" else None)
        tw, ti = tm.route(logits, K, scoring, True, n_group, topk_group, scale, bias if scoring == "sigmoid" else None)
        ref = torch.zeros(M, H, dtype=torch.double)
        for m in range(M):
            for j in range(K):
                e = int(ti[m, j])
                h = x[m].double() @ w13[e].double().T
                ref[m] += tw[m, j].double() * ((F.silu(h[:I]) * h[I:]) @ w2[e].double().T)
        assert rel_l2(from_bits(out), ref) <= 1e-2
        assert rel_l2(from_bits(out), tm.bf16_moe(x, logits, w13, w2, K, True)) <= 1e-2 or scoring == "sigmoid"


def test_forward_fp8_against_a_per_expert_loop():
    """co.forward_fp8 (with a shared expert and the caller epilogue) against a torch loop built from the
    torch oracle's fp8 quantiser and block GEMM, written independently of the C code."""
    g = torch.Generator().manual_seed(24)
    M, H, E, K, I, Is = 11, 256, 6, 2, 128, 256
    x = torch.randn(M, H, generator=g).bfloat16()
    logits = torch.randn(M, E, generator=g)
    bias = torch.randn(E, generator=g) * 0.01
    w13, s13 = tm.quantize_weight_fp8_block128(torch.randn(E, 2 * I, H, generator=g) * 0.05)
    w2, s2 = tm.quantize_weight_fp8_block128(torch.randn(E, H, I, generator=g) * 0.05)
    ws13, ss13 = tm.quantize_weight_fp8_block128(torch.randn(2 * Is, H, generator=g) * 0.05)
    ws2, ss2 = tm.quantize_weight_fp8_block128(torch.randn(H, Is, generator=g) * 0.05)
    codes = lambda t: t.view(torch.uint8).numpy()  # noqa: E731
    out_scale = 2.5
    out = co.forward_fp8(bits(x), logits.numpy(), codes(w13), s13.numpy(), codes(w2), s2.numpy(), K, "sigmoid", True, 3,
                         2, 1.0, bias.numpy(), (codes(ws13), ss13.numpy(), codes(ws2), ss2.numpy()), out_scale)

    def mlp(rows, wa, sa, wb, sb):
        q, s = tm.quant_fp8_group128(rows)
        a = tm.silu_and_mul(tm.fp8_block_gemm(q, s, wa, sa))
        q, s = tm.quant_fp8_group128(a)
        return tm.fp8_block_gemm(q, s, wb, sb)

    tw, ti = tm.route(logits, K, "sigmoid", True, 3, 2, 1.0, bias)
    ref = torch.zeros(M, H)
    for m in range(M):
        for j in range(K):
            e = int(ti[m, j])
            ref[m] += tw[m, j] * mlp(x[m:m + 1], w13[e], s13[e], w2[e], s2[e])[0].float()
    ref = (ref.bfloat16().float() * out_scale).bfloat16().float() + mlp(x, ws13, ss13, ws2, ss2).float()
    assert rel_l2(from_bits(out), ref) <= 1e-2
    no_shared = co.forward_fp8(bits(x), logits.numpy(), codes(w13), s13.numpy(), codes(w2), s2.numpy(), K, "sigmoid",
                               True, 3, 2, 1.0, bias.numpy())
    assert rel_l2(from_bits(no_shared), ref) > 0.1     # the shared expert and the factor are not optional extras


# ------------------------------------------------------------------ float16 activations (int8 path)
def test_half_conversions_match_numpy_float16():
    """Every half pattern decodes to numpy's value; f32 -> half is numpy's round-to-nearest-even cast on ties,
    subnormals, the overflow threshold, infinities and NaN."""
    allbits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    got = co.half_bits_to_f32(allbits)
    want = allbits.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.all(np.isnan(got[np.isnan(want)]))
    rng = np.random.default_rng(5)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 65536.0, 1e6, -1e6, np.inf, -np.inf, 2.0 ** -24, 2.0 ** -25,
                  2.0 ** -25 * 1.0001, 3 * 2.0 ** -25, 2.0 ** -14, 2.0 ** -14 * (1 - 2.0 ** -11), 1.0 + 2.0 ** -11,
                  1.0 + 3 * 2.0 ** -11, 1.0 + 2.0 ** -11 + 2.0 ** -20, 2047.5, 2048.5, 2049.5], np.float32),
        # every tie between neighbouring halves in [1, 2): exactly representable in f32
        (1.0 + (np.arange(1024) + 0.5) * 2.0 ** -10).astype(np.float32)])
    with np.errstate(over="ignore"):
        want_bits = vals.astype(np.float16).view(np.uint16)
    assert np.array_equal(co.f32_to_half_bits(vals), want_bits)
    assert co.f32_to_half_bits(np.array([np.nan], np.float32))[0] & 0x7c00 == 0x7c00


def _half_bits(t: torch.Tensor) -> np.ndarray:
    return t.to(torch.float16).contiguous().view(torch.int16).numpy().view(np.uint16)


def _from_half_bits(b: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(b).view(np.int16)).view(torch.float16)


def test_half_stages_closed_forms():
    """The int8 path's stages with float16 activations: quantiser, GEMM epilogue, SiLU-mul and combine (with the
    half form of the caller epilogue: the shared output scaled, not the routed sum) against numpy float16
    arithmetic written out step by step."""
    g = torch.Generator().manual_seed(31)
    x = (torch.randn(7, 96, generator=g) * 3).half()
    q, mx = co.quant_i8_rows(_half_bits(x), f16=True)
    xf = x.float().numpy()
    amax = np.abs(xf).max(1)
    assert np.array_equal(mx, amax)
    want_q = np.clip(np.rint(xf * (np.float32(127.0) / amax)[:, None]), -127, 127).astype(np.int8)
    assert np.array_equal(q, want_q)
    # GEMM epilogue: f16( (acc * a_max/127) * (w_max/127) ), SiLU-mul on the half-rounded gate and up
    rng = np.random.default_rng(32)
    E, n, k = 2, 64, 128
    lod = np.array([0, 3, 7], np.int32)
    w = rng.integers(-127, 128, (E, n, k), dtype=np.int8)
    w_max = (rng.random((E, n)) * 0.05 + 0.01).astype(np.float32)
    y, acc = co.grouped_gemm_i8(q[:, :k] if k <= 96 else np.pad(q, ((0, 0), (0, k - 96))), mx, w, w_max, lod,
                                want_acc=True, f16=True)
    qa = np.pad(q, ((0, 0), (0, k - 96)))
    for e in range(E):
        r0, r1 = lod[e], lod[e + 1]
        a64 = qa[r0:r1].astype(np.int64) @ w[e].astype(np.int64).T
        assert np.array_equal(acc[r0:r1], a64)
        deq = (a64.astype(np.float32) * (mx[r0:r1, None] / np.float32(127))) * (w_max[e][None] / np.float32(127))
        assert np.array_equal(y[r0:r1], deq.astype(np.float16).view(np.uint16))
    fused, _ = co.grouped_gemm_i8(qa, mx, w, w_max, lod, act=1, f16=True)
    assert np.array_equal(fused, co.silu_and_mul(y, f16=True))
    yt = _from_half_bits(y).float()
    silu_ref = (F.silu(yt[:, :n // 2].double()) * yt[:, n // 2:].double())
    got = _from_half_bits(fused).double()
    assert float((got - silu_ref).abs().max()) <= float(silu_ref.abs().max()) * 2 ** -10
    assert not np.array_equal(fused, co.silu_and_mul(y, f16=False))           # the dtype switch is not a no-op
    # combine: f32 accumulation over ascending k, one half rounding; epilogue routed*1 + f16(shared * s)
    M, K, H = 5, 3, 32
    rows = (torch.randn(M * K, H, generator=g) * 2).half()
    wts = torch.rand(M, K, generator=g)
    idx = torch.randperm(M * K, generator=g).int().view(M, K)
    shared = torch.randn(M, H, generator=g).half()
    s = np.float32(1.0 / 2.5)
    out = co.combine(_half_bits(rows), idx.numpy(), wts.numpy(), addend=_half_bits(shared), addend_scale=float(s),
                     f16=True)
    rf = rows.float().numpy()
    ref = np.zeros((M, H), np.float32)
    for m in range(M):
        accv = np.zeros(H, np.float32)
        for kk in range(K):
            accv = (np.float64(wts[m, kk].item()) * rf[idx[m, kk]].astype(np.float64) + accv.astype(np.float64)).astype(np.float32)  # fmaf
        routed = accv.astype(np.float16)
        sh = (shared[m].float().numpy() * s).astype(np.float16)
        ref[m] = (routed.astype(np.float32) + sh.astype(np.float32)).astype(np.float16).astype(np.float32)
    assert np.array_equal(out, ref.astype(np.float16).view(np.uint16))


def test_half_layer_against_the_torch_expert_loop():
    """co.forward_w8a8 with float16 activations against the dtype-generic torch loop run in float16, with the
    half form of the caller epilogue (models/deepseek_v2.py:286-292)."""
    x, logits, w13, w13_max, w2, w2_max, sh = _layer_inputs(24, 128, 8, 2, 64, seed=33, shared_I=64)
    xh = x.half()
    scale = 2.5
    out = co.forward_w8a8(_half_bits(xh), logits.numpy(), w13.numpy(), w13_max.numpy(), w2.numpy(), w2_max.numpy(), 2,
                          shared=tuple(t.numpy() for t in sh), shared_scale=1.0 / scale, f16=True)
    routed = tm.w8a8_moe(xh, logits, w13, w13_max, w2, w2_max, 2)
    dense = tm.w8a8_dense(xh, *sh)
    ref = routed + dense * (1.0 / scale)
    assert ref.dtype == torch.float16
    assert rel_l2(_from_half_bits(out), ref) <= 1e-2
    # bf16 and half runs of the same layer agree to within their precisions, and differ in their bits
    out_b = co.forward_w8a8(bits(x), logits.numpy(), w13.numpy(), w13_max.numpy(), w2.numpy(), w2_max.numpy(), 2)
    out_h = co.forward_w8a8(_half_bits(xh), logits.numpy(), w13.numpy(), w13_max.numpy(), w2.numpy(), w2_max.numpy(), 2,
                            f16=True)
    assert rel_l2(_from_half_bits(out_h), from_bits(out_b)) <= 2e-2


# ------------------------------------------------------------------ static and asymmetric int8
def test_quant_i8_static_known_answers_and_the_library_quantiser():
    """x / scale rounded half to even, zero point added in integers, saturation to [-128, 127]: hand-made
    answers, and torch.quantize_per_tensor (its inverse-scale product is exact for power-of-two scales)."""
    x = torch.tensor([[0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 127.0, 128.0],
                      [-128.0, -129.0, 300.0, -300.0, 3.0, 0.0, 1e30, -1e30]]).bfloat16()
    q = co.quant_i8_static(bits(x), 1.0)
    assert q.tolist() == [[0, 2, 2, 0, -2, -2, 127, 127], [-128, -128, 127, -128, 3, 0, 127, -128]]
    q = co.quant_i8_static(bits(x), 1.0, azp=5)  # the zero point moves the codes before the saturation
    assert q.tolist() == [[5, 7, 7, 5, 3, 3, 127, 127], [-123, -124, 127, -128, 8, 5, 127, -128]]
    q = co.quant_i8_static(bits(x), 0.5, azp=-100)
    assert q[0].tolist() == [-99, -97, -95, -101, -103, -105, 127, 127]
    g = torch.Generator().manual_seed(0)
    for dtype, f16 in ((torch.bfloat16, False), (torch.float16, True)):
        xr = (torch.randn(64, 96, generator=g) * 3).to(dtype)
        for scale, zp in ((0.0625, 0), (0.03125, 17), (0.125, -90)):
            ref = torch.quantize_per_tensor(xr.float(), scale, zp, torch.qint8).int_repr().numpy()
            got = co.quant_i8_static(bits(xr), scale, azp=zp if zp else None, f16=f16)
            assert np.array_equal(got, ref), (dtype, scale, zp)
    # a scale that is no power of two: the quotient is the IEEE float division, not a product with 1 / scale
    xr = (torch.randn(32, 64, generator=g) * 3).bfloat16()
    s = np.float32(0.0237)
    ref = np.clip(np.rint(xr.float().numpy() / s), -128, 127).astype(np.int8)
    assert np.array_equal(co.quant_i8_static(bits(xr), s), ref)


def test_quant_i8_rows_azp_closed_forms_and_invariants():
    """Per row: scale (max - min) / 255, zero point rint(-128 - min / scale). Rows whose answer is known in
    closed form; for random rows the minimum lands on -128, the maximum on 127 (within one code, the two
    roundings), every value is recovered within one step, and the codes are monotone in the values."""
    ramp = torch.arange(-128, 128, dtype=torch.float32)
    rows = torch.stack([ramp, ramp + 128.0, ramp * 0.5, -ramp, torch.full((256,), 3.0), torch.zeros(256)])
    q, s, z = co.quant_i8_rows_azp(bits(rows.bfloat16()))
    assert s.tolist() == [1.0, 1.0, 0.5, 1.0, 1.0, 1.0]
    assert z.tolist() == [0, -128, 0, -1, -131, -128]  # -ramp runs from -127 to 128: its zero point is -1
    assert np.array_equal(q[0], np.arange(-128, 128)) and np.array_equal(q[1], np.arange(-128, 128))
    assert np.array_equal(q[2], np.arange(-128, 128)) and np.array_equal(q[3], np.arange(-128, 128)[::-1])
    assert (q[4] == -128).all() and (q[5] == -128).all()  # a constant row: scale 1, every code rint(v) + azp
    g = torch.Generator().manual_seed(1)
    for dtype, f16 in ((torch.bfloat16, False), (torch.float16, True)):
        x = (torch.randn(200, 333, generator=g) * torch.rand(200, 1, generator=g) * 8 + torch.randn(200, 1, generator=g) * 4)
        x = x.to(dtype)
        q, s, z = co.quant_i8_rows_azp(bits(x), f16=f16)
        xf = x.float().numpy()
        lo, hi = xf.min(1), xf.max(1)
        assert np.array_equal(s, (hi - lo) / np.float32(255.0))
        assert np.array_equal(z, np.rint(np.float32(-128.0) - lo / s).astype(np.int32))
        qi = q.astype(np.int32)
        assert (np.abs(qi[np.arange(200), xf.argmin(1)] + 128) <= 1).all()
        assert (np.abs(qi[np.arange(200), xf.argmax(1)] - 127) <= 1).all()
        back = (qi - z[:, None]) * s[:, None]
        assert (np.abs(back - xf) <= s[:, None] * 1.001).all()
        order = np.argsort(xf, axis=1, kind="stable")
        assert (np.diff(np.take_along_axis(qi, order, 1), axis=1) >= 0).all()


def test_scaled_mm_azp_against_the_dequantised_product():
    """out = scale_a * scale_b * (a @ w.T - azp * sum_k w) + bias is the product of the DEQUANTISED operands,
    sum_k (a - azp) * scale_a * w * scale_b + bias: evaluated in f64 from that definition (no accumulator, no
    column sums), the oracle's 16-bit result is its rounding within one unit in the last place. Exact cases: unit
    scales and small integers. Shapes M != n != k, so a transposed operand or a zero point on the wrong axis fails."""
    g = np.random.default_rng(0)
    M, n, k = 7, 12, 40
    a = g.integers(-128, 128, (M, k), dtype=np.int8)
    w = g.integers(-128, 128, (n, k), dtype=np.int8)
    azp = g.integers(-200, 100, M).astype(np.int32)
    adj = w.astype(np.int64).sum(1).astype(np.int32)
    sa = (g.random(M) * 0.05 + 0.01).astype(np.float32)
    sb = (g.random(n) * 0.02 + 0.001).astype(np.float32)
    bias = g.normal(size=n).astype(np.float32)
    want = ((a.astype(np.float64) - azp[:, None]) * sa[:, None].astype(np.float64)) @ (w.astype(np.float64) * sb[:, None]).T
    for f16 in (False, True):
        for b in (None, bias):
            got = co.scaled_mm_azp(a, w, sa, sb, adj, azp, b, f16=f16)
            got = (from_bits(got).double() if not f16 else torch.from_numpy(got.view(np.float16).copy()).double()).numpy()
            ref = want + (0 if b is None else b.astype(np.float64))
            ulp = np.maximum(np.abs(ref), 1e-3) * (2.0 ** -10 if f16 else 2.0 ** -7)
            assert np.all(np.abs(got - ref) <= ulp)
    # a static scheme: the zero point folded into azp_adj gives what the per-token form gives with a constant azp
    z = np.int32(-37)
    per_token = co.scaled_mm_azp(a, w, sa[:1], sb, adj, np.full(M, z, np.int32))
    folded = co.scaled_mm_azp(a, w, sa[:1], sb, adj * z, None)
    assert np.array_equal(per_token, folded)
    # exact: unit scales, small integers (every partial result is an integer below 256)
    a1 = g.integers(-3, 4, (5, 6), dtype=np.int8)
    w1 = g.integers(-3, 4, (4, 6), dtype=np.int8)
    z1 = g.integers(-2, 3, 5).astype(np.int32)
    exact = (a1.astype(np.int64) - z1[:, None]) @ w1.astype(np.int64).T
    got = co.scaled_mm_azp(a1, w1, np.ones(1, np.float32), np.ones(1, np.float32), w1.astype(np.int64).sum(1), z1)
    assert np.array_equal(from_bits(got).double().numpy().astype(np.int64), exact)


def test_expert_parallel_share_of_the_unquantized_layer():
    """forward_bf16(first_expert=...) against the reference's expert-parallel loop restated in torch
    (ops/_kunlun_ops.py:655-696 with ep_rank): every share within the bf16 tolerance, exact zeros for tokens
    routed elsewhere, and the shares add up to the layer over all experts."""
    g = torch.Generator().manual_seed(3)
    M, Eg, El, K, H, I = 40, 12, 3, 3, 64, 32
    x = torch.randn(M, H, generator=g).bfloat16()
    logits = torch.randn(M, Eg, generator=g)
    w13 = (torch.randn(Eg, 2 * I, H, generator=g) * 0.1).bfloat16()
    w2 = (torch.randn(Eg, H, I, generator=g) * 0.1).bfloat16()
    _, ids = co.softmax_topk(logits.numpy(), K, True)
    total = torch.zeros(M, H, dtype=torch.float64)
    for rank in range(Eg // El):
        lo = rank * El
        got = from_bits(co.forward_bf16(bits(x), logits.numpy(), bits(w13[lo:lo + El]), bits(w2[lo:lo + El]), K,
                                        first_expert=lo))
        assert rel_l2(got, tm.bf16_moe(x, logits, w13[lo:lo + El], w2[lo:lo + El], K, True, ep_rank=rank)) <= 1e-2
        elsewhere = torch.from_numpy(~((ids >= lo) & (ids < lo + El)).any(1))
        assert elsewhere.any() and not got[elsewhere].any()
        total += got.double()
    assert rel_l2(total, from_bits(co.forward_bf16(bits(x), logits.numpy(), bits(w13), bits(w2), K)).double()) <= 1e-2
