"""GPU parity, stage by stage: every kernel is called through the C ABI (ctypes on
libkmoe.so) and compared with the C oracle on the same seeded inputs.

Bars: routing ids, sort maps, int8 codes, int32 accumulators — bit-exact.
bf16/f32 stage outputs — bit-exact too, because oracle and kernels perform the
same fixed float sequences (SiLU: the oracle looks it up in the device's table of
all 65536 16-bit arguments, which test_device_silu_table holds against the closed
form); the looser north-star tolerance (rel-L2 <= 1e-2) is asserted against the
independently written torch oracle in test_gpu_layer.py.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from conftest import bits, from_bits

pytestmark = pytest.mark.gpu

from oracle import c_oracle as co  # noqa: E402


@pytest.fixture(scope="module")
def L():
    from vllm_kunlun_amd import _lib
    return _lib


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.view(dtype)
    return t.cuda()


def sync():
    torch.cuda.synchronize()


# ------------------------------------------------------------------ routing
@pytest.mark.parametrize("M,E,K", [(32, 8, 2), (64, 128, 8), (1000, 128, 8), (7, 60, 6), (33, 384, 8), (5, 1024, 64),
                                   (1, 1, 1), (3, 65, 65 // 2)])
@pytest.mark.parametrize("renorm", [0, 1])
def test_softmax_topk(L, M, E, K, renorm):
    rng = np.random.default_rng(M * 1000 + E + K)
    logits = rng.standard_normal((M, E)).astype(np.float32)
    logits[0, : min(E, 4)] = 0.5  # exact ties: lower id must win
    w_ref, ids_ref = co.softmax_topk(logits, K, renorm)
    d_logits = dev(logits)
    w = torch.empty(M, K, dtype=torch.float32, device="cuda")
    ids = torch.empty(M, K, dtype=torch.int32, device="cuda")
    L.check(L.lib.kmoe_softmax_topk(L.ptr(d_logits), M, E, K, renorm, L.ptr(w), L.ptr(ids), L.stream()))
    sync()
    assert np.array_equal(ids.cpu().numpy(), ids_ref)
    assert np.array_equal(w.cpu().numpy().view(np.uint32), w_ref.view(np.uint32))


@pytest.mark.parametrize("M,E,K,ng,tg", [(128, 256, 8, 8, 4), (64, 384, 8, 1, 1), (17, 64, 6, 4, 2),
                                         (9, 16, 4, 8, 2), (300, 256, 8, 8, 4), (4, 1024, 8, 16, 4)])
@pytest.mark.parametrize("with_bias", [True, False])
def test_sigmoid_group_topk(L, M, E, K, ng, tg, with_bias):
    rng = np.random.default_rng(M + E + K + ng)
    logits = rng.standard_normal((M, E)).astype(np.float32)
    bias = (rng.standard_normal(E) * 0.01).astype(np.float32) if with_bias else None
    w_ref, ids_ref = co.sigmoid_group_topk_norm(logits, bias, K, ng, tg, 2.5)
    w = torch.empty(M, K, dtype=torch.float32, device="cuda")
    ids = torch.empty(M, K, dtype=torch.int32, device="cuda")
    d_logits = dev(logits)
    d_bias = None if bias is None else dev(bias)
    L.check(L.lib.kmoe_sigmoid_group_topk_norm(L.ptr(d_logits), L.ptr(d_bias), M, E, K, ng, tg, 2.5, L.ptr(w),
                                               L.ptr(ids), L.stream()))
    sync()
    assert np.array_equal(ids.cpu().numpy(), ids_ref)
    assert np.array_equal(w.cpu().numpy().view(np.uint32), w_ref.view(np.uint32))


# -------------------------------------------------------------------- align
def _run_align(L, ids_np, E):
    P = ids_np.size
    d_ids = dev(ids_np.astype(np.int32))
    moe_index = torch.full((P,), -7, dtype=torch.int32, device="cuda")
    sorted_src = torch.full((P,), -7, dtype=torch.int32, device="cuda")
    expert_m = torch.empty(E, dtype=torch.int32, device="cuda")
    lod = torch.empty(E + 1, dtype=torch.int32, device="cuda")
    nbytes = L.lib.kmoe_align_workspace_bytes(P, E)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    L.check(L.lib.kmoe_align(L.ptr(d_ids), P, E, L.ptr(moe_index), L.ptr(sorted_src), L.ptr(expert_m), L.ptr(lod),
                             L.ptr(ws), nbytes, L.stream()))
    sync()
    return moe_index.cpu().numpy(), sorted_src.cpu().numpy(), expert_m.cpu().numpy(), lod.cpu().numpy()


@pytest.mark.parametrize("P,E,kind", [(0, 8, "uniform"), (1, 8, "uniform"), (64, 8, "uniform"), (512, 128, "uniform"),
                                      (1024, 256, "uniform"), (1000, 384, "skew"), (8192, 128, "skew"),
                                      (8193, 128, "uniform"), (65536, 128, "skew"), (32768, 256, "uniform"),
                                      (40000, 1024, "onehot"), (5000, 33, "holes"),
                                      # many chunks of 2048 pairs for the three-launch path
                                      (131072, 128, "uniform"), (131073, 64, "skew"), (300000, 256, "uniform"),
                                      (140000, 1024, "holes")])
def test_align(L, P, E, kind):
    rng = np.random.default_rng(P + E)
    if kind == "uniform":
        ids = rng.integers(0, E, P)
    elif kind == "skew":
        p = np.ones(E)
        p[:: max(1, E // 8)] += 20.0
        ids = rng.choice(E, P, p=p / p.sum())
    elif kind == "onehot":
        ids = np.full(P, E - 1)
    else:  # experts that nobody picks
        ids = rng.integers(0, E // 3, P) * 3
    mi_ref, src_ref, em_ref, lod_ref = co.align(ids, E)
    mi, src, em, lod = _run_align(L, ids, E)
    assert np.array_equal(lod, lod_ref)
    assert np.array_equal(em, em_ref)
    assert np.array_equal(mi, mi_ref)
    assert np.array_equal(src, src_ref)


def test_align_skips_out_of_range_ids(L):
    ids = np.array([3, -1, 2, 99, 3, 0, 2, 3], dtype=np.int32)
    mi_ref, src_ref, em_ref, lod_ref = co.align(ids, 4)
    mi, src, em, lod = _run_align(L, ids, 4)
    assert np.array_equal(mi, mi_ref) and np.array_equal(lod, lod_ref) and np.array_equal(em, em_ref)
    assert np.array_equal(src[: lod[-1]], src_ref[: lod_ref[-1]])


@pytest.mark.parametrize("P,E,B", [(512, 128, 12), (65536, 128, 12), (7, 8, 12)])
def test_block_statistic(L, P, E, B):
    ids = np.random.default_rng(P).integers(0, E, P).astype(np.int32)
    out = torch.empty(B, E, dtype=torch.int32, device="cuda")
    L.check(L.lib.kmoe_block_statistic(L.ptr(dev(ids)), P, E, B, L.ptr(out), L.stream()))
    sync()
    got = out.cpu().numpy()
    assert np.array_equal(got, co.block_statistic(ids, E, B))
    assert np.array_equal(got.sum(0), np.bincount(ids, minlength=E))


def test_gather_rows(L):
    M, K, H, E = 37, 4, 256, 16
    x = torch.randn(M, H).bfloat16().cuda()
    ids = np.random.default_rng(0).integers(0, E, M * K).astype(np.int32)
    _, src, _, _ = co.align(ids, E)
    out = torch.empty(M * K, H, dtype=torch.bfloat16, device="cuda")
    L.check(L.lib.kmoe_gather_rows(L.ptr(x), H, L.ptr(dev(src)), M * K, K, H, L.ptr(out), H, L.stream()))
    sync()
    assert torch.equal(out.cpu(), x.cpu()[torch.from_numpy(src // K).long()])


# -------------------------------------------------------------------- quant
@pytest.mark.parametrize("R,Cc", [(1, 8), (5, 256), (64, 2048), (100, 768), (33, 7168), (3, 16384), (7, 1000),
                                  (512, 2048), (5, 20480), (2, 65536)])
def test_quant_i8_rows(L, R, Cc):
    torch.manual_seed(R + Cc)
    x = (torch.randn(R, Cc) * torch.rand(R, 1) * 4).bfloat16()
    x[0] = 0  # all-zero row
    if R > 2:
        x[1, :] = 0.5  # constant row: every element is the max
        x[2, Cc // 2] = 300.0
    q_ref, mx_ref = co.quant_i8_rows(bits(x))
    dx = x.cuda()
    q = torch.empty(R, Cc, dtype=torch.int8, device="cuda")
    mx = torch.empty(R, dtype=torch.float32, device="cuda")
    L.check(L.lib.kmoe_quant_i8_rows(L.ptr(dx), Cc, R, Cc, L.ptr(q), Cc, L.ptr(mx), L.stream()))
    sync()
    assert np.array_equal(mx.cpu().numpy().view(np.uint32), mx_ref.view(np.uint32))
    assert np.array_equal(q.cpu().numpy(), q_ref)


@pytest.mark.parametrize("R,Cc", [(1, 8), (5, 256), (100, 768), (33, 7168), (512, 2048), (2, 65536)])
@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("scale,azp", [(0.0237, None), (0.0625, 17), (0.011, -90)])
def test_quant_i8_static(L, R, Cc, half, scale, azp):
    """One scale (and zero point) for the tensor, through the C ABI and through `_C::scaled_int8_quant`: the
    oracle's codes, bit for bit (values far outside the range saturate on both sides)."""
    import vllm_kunlun_amd  # noqa: F401  (registers torch.ops._C.*)
    torch.manual_seed(R + Cc)
    x = (torch.randn(R, Cc) * 2).to(torch.float16 if half else torch.bfloat16)
    x[0, 0], x[0, 1] = 6e4, -6e4
    ref = co.quant_i8_static(bits(x), np.float32(scale), azp, f16=half)
    dx = x.cuda()
    ds = torch.tensor([scale], dtype=torch.float32, device="cuda")
    dz = None if azp is None else torch.tensor([azp], dtype=torch.int32, device="cuda")
    q = torch.empty(R, Cc, dtype=torch.int8, device="cuda")
    L.check(L.lib.kmoe_quant_i8_static(L.ptr(dx), Cc, R, Cc, L.ptr(ds), L.ptr(dz), L.ptr(q), Cc, L.act_dtype(dx),
                                       L.stream()))
    sync()
    assert np.array_equal(q.cpu().numpy(), ref)
    q2, s2, z2, static = torch.ops._C.scaled_int8_quant(dx.view(1, R, Cc), ds, dz, azp is None)
    sync()
    assert static and q2.shape == (1, R, Cc) and np.array_equal(q2.cpu().numpy()[0], ref)
    assert torch.equal(s2, ds) and (z2.numel() == 0 if azp is None else torch.equal(z2, dz))


@pytest.mark.parametrize("R,Cc", [(1, 8), (5, 256), (100, 768), (33, 7168), (7, 1000), (3, 1), (2, 65536)])
@pytest.mark.parametrize("half", [False, True])
def test_quant_i8_rows_azp(L, R, Cc, half):
    """Per-row scale and zero point (dynamic asymmetric), through the C ABI and through `_C::scaled_int8_quant`:
    codes, scales and zero points of the oracle, bit for bit; a constant row and an all-zero row included."""
    import vllm_kunlun_amd  # noqa: F401
    torch.manual_seed(R * 7 + Cc)
    x = (torch.randn(R, Cc) * torch.rand(R, 1) * 4 + torch.randn(R, 1) * 3).to(torch.float16 if half else torch.bfloat16)
    x[0] = 0
    if R > 2:
        x[1] = 0.75
    q_ref, s_ref, z_ref = co.quant_i8_rows_azp(bits(x), f16=half)
    dx = x.cuda()
    q = torch.empty(R, Cc, dtype=torch.int8, device="cuda")
    s = torch.empty(R, dtype=torch.float32, device="cuda")
    z = torch.empty(R, dtype=torch.int32, device="cuda")
    L.check(L.lib.kmoe_quant_i8_rows_azp(L.ptr(dx), Cc, R, Cc, L.ptr(q), Cc, L.ptr(s), L.ptr(z), L.act_dtype(dx),
                                         L.stream()))
    sync()
    assert np.array_equal(s.cpu().numpy().view(np.uint32), s_ref.view(np.uint32))
    assert np.array_equal(z.cpu().numpy(), z_ref)
    assert np.array_equal(q.cpu().numpy(), q_ref)
    q2, s2, z2, static = torch.ops._C.scaled_int8_quant(dx, None, None, False)
    sync()
    assert not static and s2.shape == (R, 1) and z2.shape == (R, 1) and z2.dtype == torch.int32
    assert np.array_equal(q2.cpu().numpy(), q_ref) and np.array_equal(s2.cpu().numpy().ravel(), s_ref)
    assert np.array_equal(z2.cpu().numpy().ravel(), z_ref)


def test_quant_i8_static_refusals(L):
    import vllm_kunlun_amd  # noqa: F401
    x = torch.zeros(4, 12, dtype=torch.bfloat16, device="cuda")  # 12 columns: not a multiple of 8
    s = torch.ones(1, dtype=torch.float32, device="cuda")
    with pytest.raises(Exception, match="quant_i8_static"):
        torch.ops._C.scaled_int8_quant(x, s, None, True)
    with pytest.raises(Exception, match="one float32"):
        torch.ops._C.scaled_int8_quant(torch.zeros(4, 16, dtype=torch.bfloat16, device="cuda"),
                                       torch.ones(4, dtype=torch.float32, device="cuda"), None, True)


@pytest.mark.parametrize("R,Cc", [(1, 128), (17, 2048), (64, 7168), (5, 384)])
def test_quant_fp8_group128(L, R, Cc):
    torch.manual_seed(R + Cc)
    x = (torch.randn(R, Cc) * torch.rand(R, 1) * 4).bfloat16()
    x[0, :128] = 0
    if Cc > 128:
        x[0, 130] = 2.0 ** -12
    q_ref, s_ref = co.quant_fp8_group128(bits(x))
    dx = x.cuda()
    q = torch.empty(R, Cc, dtype=torch.uint8, device="cuda")
    s = torch.empty(R, Cc // 128, dtype=torch.float32, device="cuda")
    L.check(L.lib.kmoe_quant_fp8_group128(L.ptr(dx), Cc, R, Cc, L.ptr(q), Cc, L.ptr(s), L.stream()))
    sync()
    assert np.array_equal(s.cpu().numpy().view(np.uint32), s_ref.view(np.uint32))
    assert np.array_equal(q.cpu().numpy(), q_ref)


def test_quant_fp8_every_bf16_value(L):
    """Every finite bf16 value of magnitude <= 448 (both zeros and the subnormals included), each in
    a group whose absmax is exactly 448, so that the scale is 1 and the value itself is encoded:
    the conversion instruction against the oracle's nearest-value search, code by code. A second pass
    with absmax 3.5 (scale 2^-7) puts the small values onto the e4m3 subnormal grid."""
    allbits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    vals = (allbits.astype(np.uint32) << 16).view(np.float32)
    for top in (448.0, 3.5):
        keep = allbits[np.isfinite(vals) & (np.abs(vals) <= top)]
        rows = -(-keep.size // 127)
        x = np.zeros((rows, 128), dtype=np.uint16)
        x[:, 0] = np.array([top], dtype=np.float32).view(np.uint32)[0] >> 16
        body = np.zeros(rows * 127, dtype=np.uint16)
        body[:keep.size] = keep
        x[:, 1:] = body.reshape(rows, 127)
        q_ref, s_ref = co.quant_fp8_group128(x)
        assert np.all(s_ref == np.float32(top) / np.float32(448.0))
        dx = torch.from_numpy(x.view(np.int16)).cuda()
        q = torch.empty(rows, 128, dtype=torch.uint8, device="cuda")
        s = torch.empty(rows, 1, dtype=torch.float32, device="cuda")
        L.check(L.lib.kmoe_quant_fp8_group128(L.ptr(dx), 128, rows, 128, L.ptr(q), 128, L.ptr(s), L.stream()))
        sync()
        assert np.array_equal(s.cpu().numpy().view(np.uint32), s_ref.reshape(rows, 1).view(np.uint32))
        got = q.cpu().numpy()
        assert np.array_equal(got, q_ref), np.argwhere(got != q_ref)[:5]
        assert len(np.unique(got & 0x7f)) >= 120  # nearly every code occurs


# --------------------------------------------------------------- grouped GEMM
def _gemm_case(L, E, n, k, counts, act, variant, gather, seed=0):
    """Runs one grouped GEMM on device and returns (y, acc, y_ref, acc_ref)."""
    rng = np.random.default_rng(seed)
    counts = np.asarray(counts, dtype=np.int32)
    assert counts.size == E
    lod = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    rows = int(lod[-1])
    w = rng.integers(-127, 128, (E, n, k), dtype=np.int8)
    w_max = (rng.random((E, n)) * 0.1 + 0.01).astype(np.float32)
    if gather:
        src_div = 4
        a_rows = max(1, (rows + src_div - 1) // src_div)
        row_src = rng.permutation(a_rows * src_div)[:rows].astype(np.int32)
    else:
        src_div, a_rows, row_src = 1, max(rows, 1), None
    a = rng.integers(-127, 128, (a_rows, k), dtype=np.int8)
    a_max = (rng.random(a_rows) * 4 + 0.1).astype(np.float32)
    y_ref, acc_ref = co.grouped_gemm_i8(a, a_max, w, w_max, lod, act=act, row_src=row_src, src_div=src_div,
                                        want_acc=True)
    n_out = n // 2 if act else n
    d = dict(a=dev(a), a_max=dev(a_max), w=dev(w), w_max=dev(w_max), lod=dev(lod),
             row_src=None if row_src is None else dev(row_src))
    y = torch.zeros(max(rows, 1), n_out, dtype=torch.bfloat16, device="cuda")
    acc = torch.zeros(max(rows, 1), n, dtype=torch.int32, device="cuda")
    args = L.GemmI8Args()
    args.a, args.lda, args.a_max = d["a"].data_ptr(), k, d["a_max"].data_ptr()
    args.row_src = 0 if row_src is None else d["row_src"].data_ptr()
    args.src_div = src_div
    args.w, args.w_max, args.lod = d["w"].data_ptr(), d["w_max"].data_ptr(), d["lod"].data_ptr()
    args.E, args.n, args.k, args.rows = E, n, k, rows
    args.y, args.ldy, args.acc_out = y.data_ptr(), n_out, acc.data_ptr()
    args.act, args.variant = act, variant
    L.check(L.lib.kmoe_grouped_gemm_i8(args, L.stream()))
    sync()
    return bits(y)[:rows], acc.cpu().numpy()[:rows], y_ref, acc_ref


GEMM_CASES = [
    # E, n, k, counts
    (1, 64, 256, [16]),
    (4, 64, 256, [3, 0, 17, 1]),
    (8, 128, 512, [4, 4, 0, 9, 33, 1, 0, 2]),
    (3, 96, 768, [5, 40, 7]),          # n not a multiple of the workgroup's channel span
    (2, 256, 2048, [130, 129]),
    (5, 1536, 64, [1, 2, 3, 4, 5]),    # k shorter than one 256-byte chunk
    (2, 64, 272, [20, 3]),             # k = 256 + 16: ragged last chunk
    (16, 192, 384, [0] * 15 + [300]),  # everything on one expert
]


@pytest.mark.parametrize("E,n,k,counts", GEMM_CASES)
@pytest.mark.parametrize("variant", [1, 2, 3])
@pytest.mark.parametrize("act", [0, 1])
@pytest.mark.parametrize("gather", [False, True])
def test_grouped_gemm_i8(L, E, n, k, counts, variant, act, gather):
    if act and n % 32:
        pytest.skip("SwiGLU needs n % 32 == 0")
    y, acc, y_ref, acc_ref = _gemm_case(L, E, n, k, counts, act, variant, gather, seed=E * n + k)
    assert np.array_equal(acc, acc_ref), "int32 accumulators differ"
    assert np.array_equal(y, y_ref), "bf16 outputs differ"


def test_grouped_gemm_i8_extreme_values(L):
    """All operands at +-127: the largest accumulators the path can produce."""
    E, n, k, rows = 1, 32, 7168, 16
    a = np.full((rows, k), 127, np.int8)
    a[1::2] = -127
    w = np.full((E, n, k), 127, np.int8)
    w[:, 1::2] = -127
    lod = np.array([0, rows], np.int32)
    y_ref, acc_ref = co.grouped_gemm_i8(a, np.ones(rows, np.float32), w, np.ones((E, n), np.float32), lod,
                                        want_acc=True)
    assert abs(int(acc_ref[0, 0])) == 127 * 127 * k
    d = dict(a=dev(a), a_max=torch.ones(rows, device="cuda"), w=dev(w), w_max=torch.ones(E, n, device="cuda"),
             lod=dev(lod))
    y = torch.zeros(rows, n, dtype=torch.bfloat16, device="cuda")
    acc = torch.zeros(rows, n, dtype=torch.int32, device="cuda")
    args = L.GemmI8Args()
    args.a, args.lda, args.a_max = d["a"].data_ptr(), k, d["a_max"].data_ptr()
    args.src_div = 1
    args.w, args.w_max, args.lod = d["w"].data_ptr(), d["w_max"].data_ptr(), d["lod"].data_ptr()
    args.E, args.n, args.k, args.rows = E, n, k, rows
    args.y, args.ldy, args.acc_out = y.data_ptr(), n, acc.data_ptr()
    L.check(L.lib.kmoe_grouped_gemm_i8(args, L.stream()))
    sync()
    assert np.array_equal(acc.cpu().numpy(), acc_ref)
    assert np.array_equal(bits(y), y_ref)


# -------------------------------------------------------------- elementwise
@pytest.mark.parametrize("R,I", [(1, 8), (33, 768), (512, 2048)])
def test_silu_and_mul(L, R, I):
    torch.manual_seed(R)
    y = (torch.randn(R, 2 * I) * 3).bfloat16()
    y[0, :4] = torch.tensor([0.0, -100.0, 100.0, -0.0]).bfloat16()
    ref = co.silu_and_mul(bits(y))
    out = torch.empty(R, I, dtype=torch.bfloat16, device="cuda")
    dy = y.cuda()
    L.check(L.lib.kmoe_silu_and_mul(L.ptr(dy), 2 * I, R, I, L.ptr(out), I, L.stream()))
    sync()
    assert np.array_equal(bits(out), ref)


def test_clock_probe(L):
    """kmoe_clock_probe alone on the GPU: every run is stamped; a sleep run (8 x s_sleep 127 = 8 x 64 x 127 shader
    clocks at least) reports that many s_memtime ticks or a little more, and ticks over duration lands in the range
    of clocks this part can run at. Size limits are refused."""
    n_wg, reps = 4, 64
    samples = torch.zeros(n_wg * reps * 3, dtype=torch.int64, device="cuda")
    L.check(L.lib.kmoe_clock_probe(L.ptr(samples), n_wg, reps, L.stream()))
    sync()
    r = samples.cpu().numpy().reshape(n_wg, reps, 3)
    assert (r[:, :, 0] > 0).all() and (r[:, :, 1] > 0).all() and (r[:, :, 2] > 0).all()
    assert (np.diff(r[:, :, 0], axis=1) > 0).all()  # the 100 MHz counter moves on from run to run
    sleep_ticks, sleep_ns = r[:, 1::2, 2].astype(float), r[:, 1::2, 1].astype(float) * 10.0
    assert np.median(sleep_ticks) >= 8 * 64 * 127 and np.median(sleep_ticks) < 1.2 * 8 * 64 * 127
    ghz = np.median(sleep_ticks / sleep_ns)
    assert 0.5 < ghz < 3.0, ghz
    assert L.lib.kmoe_clock_probe(L.ptr(samples), 65, reps, L.stream()) == -2  # KMOE_ERR_SHAPE
    assert L.lib.kmoe_clock_probe(None, 1, reps, L.stream()) == -1  # KMOE_ERR_NULL


@pytest.mark.parametrize("f16", [False, True], ids=["bf16", "f16"])
def test_device_silu_table(L, f16):
    """kmoe_silu_table: the device's SiLU of all 65536 16-bit arguments. Against float64 g / (1 + exp(-g)) within
    the tolerance the oracle states (c_oracle.SILU_REL_TOL), and the stand-alone silu_and_mul kernel - the same
    device function - gives exactly the table's values rounded to the activation type (up = 1), on every argument.
    Against the unrounded torch silu the rounded outputs differ by at most one 16-bit step."""
    table = torch.empty(65536, dtype=torch.float32, device="cuda")
    L.check(L.lib.kmoe_silu_table(L.ptr(table), 1 if f16 else 0, L.stream()))
    sync()
    host = table.cpu().numpy()
    worst = co.check_silu_table(f16, host)
    assert worst <= co.SILU_REL_TOL
    dt = torch.float16 if f16 else torch.bfloat16
    gate = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dt)  # every pattern once
    y = torch.cat([gate.reshape(512, 128), torch.ones(512, 128, dtype=dt)], dim=1).cuda()
    out = torch.empty(512, 128, dtype=dt, device="cuda")
    L.check(L.lib.kmoe_silu_and_mul_dt(L.ptr(y), 256, 512, 128, L.ptr(out), 128, 1 if f16 else 0, L.stream()))
    sync()
    want = torch.from_numpy(host).to(dt).reshape(512, 128)  # torch rounds to nearest even, as the kernels do
    finite = torch.isfinite(gate.float()).reshape(512, 128)
    got = out.cpu()
    assert torch.equal(got[finite].view(torch.int16), want[finite].view(torch.int16))
    # one 16-bit step at most from the rounded closed form
    # (where the result is far below the type's normal range - arguments below -80 - "as good as zero" is the bar)
    ref = torch.nn.functional.silu(gate.float().double()).to(dt).reshape(512, 128)
    usual = finite & (gate.float() >= -80.0).reshape(512, 128)
    step = (got[usual].view(torch.int16).int() - ref[usual].view(torch.int16).int()).abs()
    assert int(step.max()) <= 1
    assert float(got[finite & ~usual].float().abs().max()) <= 1e-30


@pytest.mark.parametrize("M,K,H", [(1, 1, 8), (64, 8, 2048), (33, 6, 7168), (128, 8, 512)])
@pytest.mark.parametrize("epilogue", [False, True])
def test_combine(L, M, K, H, epilogue):
    torch.manual_seed(M + K)
    P = M * K
    x = torch.randn(P, H).bfloat16()
    w = torch.rand(M, K)
    dq = torch.rand(M, K) + 0.5
    perm = torch.randperm(P).int()
    addend = torch.randn(M, H).bfloat16() if epilogue else None
    scale = 2.5 if epilogue else 1.0
    ref = co.combine(bits(x), perm.numpy(), w.numpy(), dq.numpy(), scale, None if addend is None else bits(addend))
    out = torch.empty(M, H, dtype=torch.bfloat16, device="cuda")
    d = [t.cuda() for t in (x, perm, w, dq)]
    dadd = None if addend is None else addend.cuda()
    L.check(L.lib.kmoe_combine(L.ptr(d[0]), H, L.ptr(d[1]), L.ptr(d[2]), L.ptr(d[3]), M, K, H, scale, L.ptr(dadd), H,
                               L.ptr(out), H, L.stream()))
    sync()
    assert np.array_equal(bits(out), ref)


# ------------------------------------------- tiled weights / chunked activations
def _tile_ref(w):
    """numpy restatement of the 1 KB block layout: [E][n/16][k/64][g(4)][c(16)][16]."""
    E, n, k = w.shape
    return np.ascontiguousarray(w.reshape(E, n // 16, 16, k // 64, 4, 16).transpose(0, 1, 3, 4, 2, 5))


@pytest.mark.parametrize("E,n,k", [(1, 16, 64), (3, 48, 192), (2, 1536, 2048)])
def test_tile_weights(L, E, n, k):
    w = np.random.default_rng(E + n).integers(-128, 128, (E, n, k), dtype=np.int8)
    src = dev(w)
    dst = torch.empty_like(src)
    L.check(L.lib.kmoe_tile_weights_i8(L.ptr(src), L.ptr(dst), E, n, k, L.stream()))
    sync()
    assert np.array_equal(dst.cpu().numpy().reshape(-1), _tile_ref(w).reshape(-1))
    assert L.lib.kmoe_tile_weights_i8(L.ptr(src), L.ptr(src), E, n, k, L.stream()) == -2  # in place is refused


@pytest.mark.parametrize("R,Cc", [(1, 64), (64, 2048), (100, 768), (33, 7168), (512, 2048), (5, 20480), (2, 65536)])
def test_quant_i8_rows_chunked(L, R, Cc):
    torch.manual_seed(R + Cc)
    x = (torch.randn(R, Cc) * 3).bfloat16()
    x[0] = 0
    q_ref, mx_ref = co.quant_i8_rows(bits(x))
    dx = x.cuda()
    q = torch.empty(Cc // 64, R, 64, dtype=torch.int8, device="cuda")
    mx = torch.empty(R, dtype=torch.float32, device="cuda")
    L.check(L.lib.kmoe_quant_i8_rows_chunked(L.ptr(dx), Cc, R, Cc, L.ptr(q), L.ptr(mx), L.stream()))
    sync()
    assert np.array_equal(mx.cpu().numpy(), mx_ref)
    assert np.array_equal(q.cpu().numpy().transpose(1, 0, 2).reshape(R, Cc), q_ref)


def _gemm_layout_case(L, E, n, k, counts, act, variant, gather, chunked, seed=0):
    rng = np.random.default_rng(seed)
    counts = np.asarray(counts, dtype=np.int32)
    lod = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    rows = int(lod[-1])
    w = rng.integers(-127, 128, (E, n, k), dtype=np.int8)
    w_max = (rng.random((E, n)) * 0.1 + 0.01).astype(np.float32)
    if gather:
        src_div = 4
        a_rows = max(1, (rows + src_div - 1) // src_div)
        row_src = rng.permutation(a_rows * src_div)[:rows].astype(np.int32)
    else:
        src_div, a_rows, row_src = 1, max(rows, 1), None
    a = rng.integers(-127, 128, (a_rows, k), dtype=np.int8)
    a_max = (rng.random(a_rows) * 4 + 0.1).astype(np.float32)
    y_ref, acc_ref = co.grouped_gemm_i8(a, a_max, w, w_max, lod, act=act, row_src=row_src, src_div=src_div,
                                        want_acc=True)
    n_out = n // 2 if act else n
    a_dev = dev(np.ascontiguousarray(a.reshape(a_rows, k // 64, 64).transpose(1, 0, 2))) if chunked else dev(a)
    d = dict(a=a_dev, a_max=dev(a_max), w=dev(_tile_ref(w)), w_max=dev(w_max), lod=dev(lod),
             row_src=None if row_src is None else dev(row_src))
    y = torch.zeros(max(rows, 1), n_out, dtype=torch.bfloat16, device="cuda")
    acc = torch.zeros(max(rows, 1), n, dtype=torch.int32, device="cuda")
    args = L.GemmI8Args()
    args.a, args.lda, args.a_max = d["a"].data_ptr(), k, d["a_max"].data_ptr()
    args.row_src = 0 if row_src is None else d["row_src"].data_ptr()
    args.src_div = src_div
    args.w, args.w_max, args.lod = d["w"].data_ptr(), d["w_max"].data_ptr(), d["lod"].data_ptr()
    args.E, args.n, args.k, args.rows = E, n, k, rows
    args.y, args.ldy, args.acc_out = y.data_ptr(), n_out, acc.data_ptr()
    args.act, args.variant = act, variant
    args.w_layout = L.KMOE_W_TILED
    args.a_layout = L.KMOE_A_CHUNKED if chunked else L.KMOE_A_ROWMAJOR
    args.a_rows = a_rows
    L.check(L.lib.kmoe_grouped_gemm_i8(args, L.stream()))
    sync()
    assert np.array_equal(acc.cpu().numpy()[:rows], acc_ref), "int32 accumulators differ"
    assert np.array_equal(bits(y)[:rows], y_ref), "bf16 outputs differ"


TILED_CASES = [
    (1, 64, 256, [16]),
    (4, 64, 256, [3, 0, 17, 1]),
    (8, 128, 512, [4, 4, 0, 9, 33, 1, 0, 2]),
    (3, 96, 768, [5, 40, 7]),
    (2, 256, 2048, [130, 129]),
    (5, 1536, 64, [1, 2, 3, 4, 5]),
    (2, 32, 320, [20, 3]),
    (16, 192, 384, [0] * 15 + [300]),
]

# k % 4096 == 0: the waves of the streaming kernel walk K from rotated start steps (same sums)
ROTATED_K_CASES = [(3, 64, 4096, [5, 0, 18]), (2, 96, 8192, [3, 40])]


@pytest.mark.parametrize("E,n,k,counts", TILED_CASES + ROTATED_K_CASES)
@pytest.mark.parametrize("variant", [1, 2, 4, 8])
@pytest.mark.parametrize("act", [0, 1])
@pytest.mark.parametrize("gather", [False, True])
def test_stream_gemm_i8(L, E, n, k, counts, variant, act, gather):
    """Weight-streaming kernel: tiled weights x chunk-major activations."""
    _gemm_layout_case(L, E, n, k, counts, act, variant, gather, chunked=True, seed=E * n + k)


# more K lengths (1..7 chunks of 128: every remainder of both ring periods) and a case with more
# work items than persistent workgroups (every workgroup walks several tiles, ragged experts)
PERSISTENT_CASES = TILED_CASES + [
    (2, 64, 128, [5, 131]),
    (2, 96, 640, [140, 3]),
    (3, 64, 896, [1, 260, 17]),
    (64, 2048, 256, [((37 * i) % 290) for i in range(64)]),
    # 9 and 11 chunks (one and three past the 4-chunk period of the activation ring); hundreds of
    # experts (several passes of the 64-lane expert search), most of them empty
    (40, 512, 1152, [((53 * i) % 400) for i in range(40)]),
    (300, 256, 1408, [(129 if i % 7 == 0 else (i % 3)) for i in range(300)]),
    # an odd number of 64-byte steps (k % 128 == 64): the half chunk at every position of the ring
    (3, 64, 192, [1, 260, 17]),
    (2, 96, 448, [140, 3]),
    (4, 128, 576, [70, 0, 129, 5]),
    (2, 64, 704, [33, 200]),
    (8, 4096, 192, [((97 * i) % 300) for i in range(8)]),
    # experts that end exactly at the last row of a 128-, 192- or 256-row tile, one row before and one row past it,
    # and experts that leave whole pairs of row fragments of a wide tile without rows
    (12, 128, 384, [127, 128, 129, 191, 192, 193, 255, 256, 257, 31, 33, 65]),
    # variant 17 launches a wide-tile and a 128-row-tile kernel and the row counts decide on the device which of
    # them works: even counts (the wide one), and counts of which every fourth overflows the wide tile (the other)
    (20, 256, 256, [130 + (7 * i) % 25 for i in range(20)]),
    (20, 256, 256, [(260 if i % 4 == 0 else 95) + (7 * i) % 25 for i in range(20)]),
    # experts of more than 3 MiB of weights list their items channel block by channel block, smaller ones (every
    # case above) m-tile by m-tile: several m-tiles and channel blocks per expert in the first order
    (2, 2048, 2048, [300, 140]),
]


@pytest.mark.parametrize("E,n,k,counts", PERSISTENT_CASES)
@pytest.mark.parametrize("variant", [1, 2, 3, 5, 6, 7, 9, 11, 12, 13, 17, 18, 19, 22])
@pytest.mark.parametrize("act", [0, 1])
def test_lds_gemm_i8_with_tiled_weights(L, E, n, k, counts, variant, act):
    """LDS-staged kernels reading tiled weights and row-major activations. Variants 1-3: small
    tiles; 5-7: the persistent 128-row-tile kernel (6: 256-channel tiles, 7: 128-channel tiles
    with the deep weight ring), 19 / 18 / 22: 128-, 192-, 256-row wide tiles (eight waves side by side along the
    channels, row fragments without rows skipped pair by pair), 17: a wide tile or 128-row tiles, decided on the
    device, 5: the default, 12: sibling m-tiles paced against each other through the progress board)."""
    if variant >= 5 and k < 128:
        pytest.skip("the persistent kernel takes k >= 128")
    if variant < 5 and E >= 40:
        pytest.skip("large case: persistent kernel only")
    _gemm_layout_case(L, E, n, k, counts, act, variant, True, chunked=False, seed=E * n + k + 7)


def test_spare_cus_keeps_the_bits(L):
    """KMOE_SPARE_CUS (read once per process, hence a child process): the persistent tile kernels sized for half
    the CUs walk the same items in another distribution and must produce the same bits."""
    import os
    import subprocess
    import sys
    code = r"""
import sys, zlib
sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[2])
import numpy as np, torch, ctypes
from vllm_kunlun_amd import _lib as L
rng = np.random.default_rng(5)
E, n, k, counts = 6, 512, 1024, [130, 0, 190, 17, 300, 64]
lod = torch.tensor(np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)).cuda(); P = int(sum(counts))
w = torch.tensor(rng.integers(-127, 128, (E, n, k), dtype=np.int8)).cuda(); wt = torch.empty_like(w)
L.check(L.lib.kmoe_tile_weights_i8(w.data_ptr(), wt.data_ptr(), E, n, k, L.stream()))
wmax = torch.tensor((rng.random((E, n)) + 0.1).astype(np.float32)).cuda()
a = torch.tensor(rng.integers(-127, 128, (P, k), dtype=np.int8)).cuda()
amax = torch.tensor((rng.random(P) + 0.1).astype(np.float32)).cuda()
for variant in (18, 6, 12):
    y = torch.zeros(P, n // 2, dtype=torch.bfloat16, device="cuda")
    g = L.GemmI8Args()
    g.a, g.lda, g.a_max, g.src_div = a.data_ptr(), k, amax.data_ptr(), 1
    g.w, g.w_max, g.lod = wt.data_ptr(), wmax.data_ptr(), lod.data_ptr()
    g.E, g.n, g.k, g.rows = E, n, k, P
    g.y, g.ldy, g.act, g.variant, g.w_layout = y.data_ptr(), n // 2, 1, variant, 1
    L.check(L.lib.kmoe_grouped_gemm_i8(ctypes.byref(g), L.stream()))
    torch.cuda.synchronize()
    print(variant, zlib.crc32(y.cpu().view(torch.int16).numpy().tobytes()))
"""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    sums = []
    for spare in ("0", "128"):
        env = dict(os.environ, KMOE_SPARE_CUS=spare)
        out = subprocess.run([sys.executable, "-c", code, root, os.path.join(root, "vllm-kunlun_amd")], env=env,
                             capture_output=True, text=True, timeout=110)
        assert out.returncode == 0, out.stderr[-2000:]
        sums.append(out.stdout.split())
    assert len(sums[0]) == 6 and sums[0] == sums[1], sums
