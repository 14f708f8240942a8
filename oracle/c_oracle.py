"""ctypes/numpy front end of oracle/libmoe_oracle.so — TEST INFRASTRUCTURE.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import
this. Every function takes and returns numpy arrays (bf16 as uint16 bit
patterns) and forwards to the C restatement in moe_oracle.c, whose header
states what it follows in the reference and what pins it.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmoe_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_exp.restype = C.c_float
        _lib.orc_exp.argtypes = [C.c_float]
        _lib.orc_sigmoid.restype = C.c_float
        _lib.orc_sigmoid.argtypes = [C.c_float]
        _lib.orc_silu.restype = C.c_float
        _lib.orc_silu.argtypes = [C.c_float]
        _lib.orc_set_silu_table.restype = None
        _lib.orc_set_silu_table.argtypes = [C.c_int, C.c_void_p]
        _lib.orc_f32_to_e4m3fn.restype = C.c_uint8
        _lib.orc_f32_to_e4m3fn.argtypes = [C.c_float]
        _lib.orc_e4m3fn_to_f32.restype = C.c_float
        _lib.orc_e4m3fn_to_f32.argtypes = [C.c_uint8]
    return _lib


def _p(a):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be contiguous"
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


# -- bf16 helpers (bit patterns in uint16) -----------------------------------
def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = u + 0x7FFF + ((u >> 16) & 1)
    return (u >> 16).astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# -- scalar functions ---------------------------------------------------------
def _dtype(f16: bool) -> None:
    """Selects what the 16-bit activation tensors of the int8 path hold for the next call: bf16 or IEEE half."""
    lib().orc_set_act_dtype(1 if f16 else 0)


def f32_to_half_bits(x: np.ndarray) -> np.ndarray:
    fn = lib().orc_f32_to_half
    fn.restype, fn.argtypes = C.c_uint16, [C.c_float]
    return np.array([fn(float(v)) for v in np.asarray(x, np.float32).ravel()], np.uint16).reshape(np.shape(x))


def half_bits_to_f32(b: np.ndarray) -> np.ndarray:
    fn = lib().orc_half_to_f32
    fn.restype, fn.argtypes = C.c_float, [C.c_uint16]
    return np.array([fn(int(v)) for v in np.asarray(b, np.uint16).ravel()], np.float32).reshape(np.shape(b))


def exp(x: np.ndarray) -> np.ndarray:
    f = lib().orc_exp
    return np.array([f(float(v)) for v in np.asarray(x, dtype=np.float32).ravel()], dtype=np.float32).reshape(np.shape(x))


def sigmoid(x: np.ndarray) -> np.ndarray:
    f = lib().orc_sigmoid
    return np.array([f(float(v)) for v in np.asarray(x, dtype=np.float32).ravel()], dtype=np.float32).reshape(np.shape(x))


def silu(x: np.ndarray) -> np.ndarray:
    f = lib().orc_silu
    return np.array([f(float(v)) for v in np.asarray(x, dtype=np.float32).ravel()], dtype=np.float32).reshape(np.shape(x))


# -- the device's SiLU table ----------------------------------------------------
# The layer applies SiLU to gate values rounded to the 16-bit activation type: 65536 possible arguments per type.
# The product computes it with the GPU's exp2 / reciprocal instructions, whose bits no CPU sequence reproduces, so
# a GPU test fetches the product's table of all 65536 results (kmoe_silu_table), holds it against the closed form
# here, and installs it: from then on every oracle function that applies SiLU uses the device's values.
SILU_REL_TOL = 4e-6    # against float64 g / (1 + exp(-g)); measured on MI355X: 4.2e-7 at most
SILU_ABS_TOL = 2e-36   # results below the normal range


def act_values(f16: bool) -> np.ndarray:
    """float32 value of every 16-bit activation pattern 0..65535."""
    h = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    return h.view(np.float16).astype(np.float32) if f16 else bf16_bits_to_f32(h)


def check_silu_table(f16: bool, table: np.ndarray) -> float:
    """Holds a device SiLU table against float64 g / (1 + exp(-g)) on every finite argument; returns the largest
    relative error seen. Raises AssertionError beyond SILU_REL_TOL / SILU_ABS_TOL, or unless silu(+inf) = +inf and
    silu(-inf) is (as good as) zero."""
    table = np.asarray(table, dtype=np.float32)
    assert table.shape == (65536,)
    with np.errstate(invalid="ignore"):
        g = act_values(f16).astype(np.float64)
    fin = np.isfinite(g)
    with np.errstate(over="ignore"):
        want = g[fin] / (1.0 + np.exp(-g[fin]))
    got = table[fin].astype(np.float64)
    err = np.abs(got - want)
    ok = err <= SILU_REL_TOL * np.abs(want) + SILU_ABS_TOL
    assert ok.all(), (f"device SiLU table ({'f16' if f16 else 'bf16'}): {np.count_nonzero(~ok)} entries beyond tolerance, "
                      f"worst at g={g[fin][np.argmax(err / (np.abs(want) + 1e-30))]!r}")
    assert np.array_equal(np.signbit(got[want != 0]), np.signbit(want[want != 0]))
    inf = np.isinf(g)
    assert (table[inf & (g > 0)] == np.inf).all() and (np.abs(table[inf & (g < 0)]) <= SILU_ABS_TOL).all()
    big = np.abs(want) > 1e-30
    return float((err[big] / np.abs(want[big])).max())


def set_silu_table(f16: bool, table) -> None:
    """Installs (or, with None, removes) the SiLU table of one activation type."""
    if table is None:
        lib().orc_set_silu_table(1 if f16 else 0, None)
        return
    t = _c(table, np.float32)
    assert t.shape == (65536,)
    lib().orc_set_silu_table(1 if f16 else 0, _p(t))


def install_device_silu(fetch) -> dict:
    """fetch(f16) -> the device's SiLU table for that activation type (65536 float32, e.g. from the product's
    kmoe_silu_table). Each table is held against the closed form (check_silu_table) and installed; returns the
    largest relative error per type."""
    worst = {}
    for f16 in (False, True):
        table = np.asarray(fetch(f16), dtype=np.float32)
        worst["f16" if f16 else "bf16"] = check_silu_table(f16, table)
        set_silu_table(f16, table)
    return worst


# -- stages -------------------------------------------------------------------
def softmax_topk(logits, K, renorm):
    logits = _c(logits, np.float32)
    M, E = logits.shape
    w = np.empty((M, K), np.float32)
    ids = np.empty((M, K), np.int32)
    lib().orc_softmax_topk(_p(logits), M, E, K, int(bool(renorm)), _p(w), _p(ids))
    return w, ids


def sigmoid_group_topk_norm(logits, bias, K, n_group, topk_group, scale):
    logits = _c(logits, np.float32)
    bias = None if bias is None else _c(bias, np.float32)
    M, E = logits.shape
    w = np.empty((M, K), np.float32)
    ids = np.empty((M, K), np.int32)
    lib().orc_sigmoid_group_topk_norm(_p(logits), _p(bias), M, E, K, int(n_group or 1), int(topk_group or 1),
                                      C.c_float(scale), _p(w), _p(ids))
    return w, ids


def align(ids, E):
    ids = _c(ids, np.int32).ravel()
    P = ids.size
    moe_index = np.empty(P, np.int32)
    sorted_src = np.full(P, -1, np.int32)
    expert_m = np.empty(E, np.int32)
    lod = np.empty(E + 1, np.int32)
    lib().orc_align(_p(ids), P, E, _p(moe_index), _p(sorted_src), _p(expert_m), _p(lod))
    return moe_index, sorted_src, expert_m, lod


def block_statistic(ids, E, n_blocks):
    ids = _c(ids, np.int32).ravel()
    out = np.empty((n_blocks, E), np.int32)
    lib().orc_block_statistic(_p(ids), ids.size, E, n_blocks, _p(out))
    return out


def quant_i8_rows(x_bits, f16=False):
    _dtype(f16)
    x_bits = _c(x_bits, np.uint16)
    R, Cc = x_bits.shape
    q = np.empty((R, Cc), np.int8)
    mx = np.empty(R, np.float32)
    lib().orc_quant_i8_rows(_p(x_bits), C.c_int64(Cc), R, Cc, _p(q), C.c_int64(Cc), _p(mx))
    return q, mx


def quant_i8_static(x_bits, scale, azp=None, f16=False):
    """One scale (and zero point) for the tensor: codes int8 [R,C]."""
    _dtype(f16)
    x_bits = _c(x_bits, np.uint16)
    R, Cc = x_bits.shape
    q = np.zeros((R, Cc), np.int8)
    lib().orc_quant_i8_static(_p(x_bits), C.c_int64(Cc), R, Cc, C.c_float(float(scale)), 0 if azp is None else 1,
                              0 if azp is None else int(azp), _p(q), C.c_int64(Cc))
    return q


def scaled_mm_azp(a, w, scale_a, scale_b, azp_adj, azp=None, bias=None, f16=False):
    """int8 a [M,k] x w [n,k] with the asymmetric-activation epilogue: 16-bit patterns [M,n]."""
    _dtype(f16)
    a, w = _c(a, np.int8), _c(w, np.int8)
    M, k = a.shape
    n = w.shape[0]
    scale_a, scale_b = _c(scale_a, np.float32).ravel(), _c(scale_b, np.float32).ravel()
    azp_adj = None if azp_adj is None else _c(azp_adj, np.int32).ravel()
    assert scale_a.size in (1, M) and scale_b.size in (1, n) and (azp_adj is None or azp_adj.size == n)
    azp = None if azp is None else _c(azp, np.int32).ravel()
    bias = None if bias is None else _c(bias, np.float32).ravel()
    out = np.zeros((M, n), np.uint16)
    lib().orc_scaled_mm_azp(_p(a), _p(w), M, n, k, _p(scale_a), int(scale_a.size == M),
                            _p(scale_b), int(scale_b.size == n), None if azp_adj is None else _p(azp_adj), None if azp is None else _p(azp),
                            None if bias is None else _p(bias), _p(out))
    return out


def quant_i8_rows_azp(x_bits, f16=False):
    """Per-row scale and zero point: (codes int8 [R,C], scale f32 [R], azp int32 [R])."""
    _dtype(f16)
    x_bits = _c(x_bits, np.uint16)
    R, Cc = x_bits.shape
    q = np.zeros((R, Cc), np.int8)
    s = np.zeros(R, np.float32)
    z = np.zeros(R, np.int32)
    lib().orc_quant_i8_rows_azp(_p(x_bits), C.c_int64(Cc), R, Cc, _p(q), C.c_int64(Cc), _p(s), _p(z))
    return q, s, z


def quant_fp8_group128(x_bits, f16=False):
    _dtype(f16)
    x_bits = _c(x_bits, np.uint16)
    R, Cc = x_bits.shape
    q = np.empty((R, Cc), np.uint8)
    s = np.empty((R, Cc // 128), np.float32)
    lib().orc_quant_fp8_group128(_p(x_bits), C.c_int64(Cc), R, Cc, _p(q), C.c_int64(Cc), _p(s))
    return q, s


def grouped_gemm_i8(a, a_max, w, w_max, lod, act=0, row_src=None, src_div=1, want_acc=False, want_y=True, f16=False):
    _dtype(f16)
    a = _c(a, np.int8)
    a_max = _c(a_max, np.float32).ravel()
    w = _c(w, np.int8)
    w_max = _c(w_max, np.float32).reshape(w.shape[0], w.shape[1])
    lod = _c(lod, np.int32)
    E, n, k = w.shape
    rows = int(lod[-1])
    row_src = None if row_src is None else _c(row_src, np.int32)
    n_out = n // 2 if act else n
    y = np.zeros((rows, n_out), np.uint16) if want_y else None
    acc = np.zeros((rows, n), np.int32) if want_acc else None
    lib().orc_grouped_gemm_i8(_p(a), C.c_int64(a.shape[1]), _p(a_max), _p(row_src), int(src_div), _p(w), _p(w_max),
                              _p(lod), E, n, k, _p(y), C.c_int64(n_out), _p(acc), int(act))
    return y, acc


def silu_and_mul(y_bits, f16=False):
    _dtype(f16)
    y_bits = _c(y_bits, np.uint16)
    R, two_i = y_bits.shape
    out = np.empty((R, two_i // 2), np.uint16)
    lib().orc_silu_and_mul(_p(y_bits), C.c_int64(two_i), R, two_i // 2, _p(out), C.c_int64(two_i // 2))
    return out


def combine(x_bits, moe_index, topk_w, dq=None, out_scale=1.0, addend=None, addend_scale=1.0, f16=False):
    _dtype(f16)
    x_bits = _c(x_bits, np.uint16)
    topk_w = _c(topk_w, np.float32)
    M, K = topk_w.shape
    H = x_bits.shape[1]
    moe_index = _c(moe_index, np.int32).reshape(M, K)
    dq = None if dq is None else _c(dq, np.float32)
    addend = None if addend is None else _c(addend, np.uint16)
    out = np.empty((M, H), np.uint16)
    lib().orc_combine(_p(x_bits), C.c_int64(H), _p(moe_index), _p(topk_w), _p(dq), M, K, H, C.c_float(out_scale),
                      _p(addend), C.c_int64(H), C.c_float(addend_scale), _p(out), C.c_int64(H))
    return out


def forward_w8a8(x_bits, logits, w13, w13_max, w2, w2_max, K, scoring="softmax", renormalize=True, n_group=1,
                 topk_group=1, routed_scale=1.0, bias=None, shared=None, out_scale=1.0, intermediates=False,
                 shared_scale=1.0, f16=False):
    """Whole layer. `shared` = (ws13, ws13_max, ws2, ws2_max) or None; f16: x and out hold IEEE half patterns.
    Returns out bits [M,H], plus a dict of intermediates when asked."""
    _dtype(f16)
    x_bits = _c(x_bits, np.uint16)
    logits = _c(logits, np.float32)
    w13 = _c(w13, np.int8)
    w2 = _c(w2, np.int8)
    E, two_i, H = w13.shape
    I = two_i // 2
    M = x_bits.shape[0]
    P = M * K
    w13_max = _c(w13_max, np.float32).reshape(E, two_i)
    w2_max = _c(w2_max, np.float32).reshape(E, H)
    bias = None if bias is None else _c(bias, np.float32)
    if shared is not None:
        ws13, ws13_max, ws2, ws2_max = shared
        ws13 = _c(ws13, np.int8)
        ws2 = _c(ws2, np.int8)
        ws13_max = _c(ws13_max, np.float32).ravel()
        ws2_max = _c(ws2_max, np.float32).ravel()
        Is = ws13.shape[0] // 2
    else:
        ws13 = ws13_max = ws2 = ws2_max = None
        Is = 0
    out = np.empty((M, H), np.uint16)
    inter = {}
    if intermediates:
        inter = dict(topk_w=np.empty((M, K), np.float32), topk_ids=np.empty((M, K), np.int32),
                     moe_index=np.empty(P, np.int32), lod=np.empty(E + 1, np.int32),
                     actq=np.empty((P, I), np.int8), actmax=np.empty(P, np.float32),
                     down=np.empty((P, H), np.uint16))
    g = inter.get
    lib().orc_forward_w8a8(M, H, E, K, I, 0 if scoring == "softmax" else 1, int(bool(renormalize)), int(n_group or 1),
                           int(topk_group or 1), C.c_float(routed_scale), _p(logits), _p(bias), _p(x_bits), _p(w13),
                           _p(w13_max), _p(w2), _p(w2_max), Is, _p(ws13), _p(ws13_max), _p(ws2), _p(ws2_max),
                           C.c_float(out_scale), C.c_float(shared_scale), _p(out), _p(g("topk_w")), _p(g("topk_ids")), _p(g("moe_index")),
                           _p(g("lod")), _p(g("actq")), _p(g("actmax")), _p(g("down")))
    return (out, inter) if intermediates else out


def router_gemm(x_bits, w_bits, f16=False):
    """(logits f32 [M,E], abs_sum f32 [M,E]): x bits [M,H], w bits [E,H], both bf16 (or both half)."""
    _dtype(f16)
    x_bits = _c(x_bits, np.uint16)
    w_bits = _c(w_bits, np.uint16)
    M, H = x_bits.shape
    E = w_bits.shape[0]
    logits = np.zeros((M, E), np.float32)
    abs_sum = np.zeros((M, E), np.float32)
    lib().orc_router_gemm(_p(x_bits), C.c_int64(H), _p(w_bits), M, H, E, _p(logits), _p(abs_sum))
    return logits, abs_sum


def grouped_gemm_bf16(a_bits, w_bits, lod, act=0, row_src=None, src_div=1, f16=False):
    """f16: operands and result hold IEEE half patterns instead of bf16."""
    _dtype(f16)
    a_bits = _c(a_bits, np.uint16)
    w_bits = _c(w_bits, np.uint16)
    lod = _c(lod, np.int32)
    E, n, k = w_bits.shape
    rows = int(lod[-1])
    row_src = None if row_src is None else _c(row_src, np.int32)
    n_out = n // 2 if act else n
    y = np.zeros((rows, n_out), np.uint16)
    lib().orc_grouped_gemm_bf16(_p(a_bits), C.c_int64(a_bits.shape[1]), _p(row_src), int(src_div), _p(w_bits),
                                _p(lod), E, n, k, _p(y), C.c_int64(n_out), int(act))
    return y


def grouped_gemm_fp8(a, a_scale, w, w_scale, lod, act=0, row_src=None, src_div=1, f16=False):
    _dtype(f16)
    a = _c(a, np.uint8)
    w = _c(w, np.uint8)
    a_scale = _c(a_scale, np.float32)
    w_scale = _c(w_scale, np.float32)
    lod = _c(lod, np.int32)
    E, n, k = w.shape
    rows = int(lod[-1])
    row_src = None if row_src is None else _c(row_src, np.int32)
    n_out = n // 2 if act else n
    y = np.zeros((rows, n_out), np.uint16)
    lib().orc_grouped_gemm_fp8(_p(a), C.c_int64(a.shape[1]), _p(a_scale), _p(row_src), int(src_div), _p(w),
                               _p(w_scale), _p(lod), E, n, k, _p(y), C.c_int64(n_out), int(act))
    return y


def _route(logits, K, scoring, renormalize, n_group, topk_group, routed_scale, bias):
    if scoring == "softmax":
        return softmax_topk(logits, K, renormalize)
    return sigmoid_group_topk_norm(logits, bias, K, n_group, topk_group, routed_scale)


def dequant_w4_bf16(packed, scale_bits, group_size, f16=False):
    """packed uint8 [..., k/2], scale bf16 bits [..., k/group_size] -> bf16 bits [..., k]; f16: scales and result
    hold IEEE half patterns (the reference's own dtype for this step)."""
    _dtype(f16)
    packed = _c(packed, np.uint8)
    scale_bits = _c(scale_bits, np.uint16)
    k = packed.shape[-1] * 2
    rows = int(np.prod(packed.shape[:-1]))
    out = np.zeros((*packed.shape[:-1], k), np.uint16)
    lib().orc_dequant_w4_bf16(_p(packed), _p(scale_bits), C.c_int64(rows), k, int(group_size), _p(out))
    return out


def swigluoai_and_mul(y_bits, alpha=1.702, limit=7.0):
    y_bits = _c(y_bits, np.uint16)
    R, two_i = y_bits.shape
    out = np.zeros((R, two_i // 2), np.uint16)
    lib().orc_swigluoai_and_mul(_p(y_bits), C.c_int64(two_i), R, two_i // 2, C.c_float(alpha), C.c_float(limit), _p(out),
                                C.c_int64(two_i // 2))
    return out


def grouped_gemm_bf16_bias(a_bits, w_bits, bias_bits, lod, act=0, row_src=None, src_div=1, alpha=1.702, limit=7.0):
    """The expert-bias branch: act 0 (none) or 2 (gpt-oss activation over interleaved columns)."""
    a_bits = _c(a_bits, np.uint16)
    w_bits = _c(w_bits, np.uint16)
    bias_bits = None if bias_bits is None else _c(bias_bits, np.uint16)
    lod = _c(lod, np.int32)
    E, n, k = w_bits.shape
    rows = int(lod[-1])
    row_src = None if row_src is None else _c(row_src, np.int32)
    n_out = n // 2 if act == 2 else n
    y = np.zeros((rows, n_out), np.uint16)
    lib().orc_grouped_gemm_bf16_bias(_p(a_bits), C.c_int64(a_bits.shape[1]), _p(row_src), int(src_div), _p(w_bits),
                                     _p(bias_bits), _p(lod), E, n, k, _p(y), C.c_int64(n_out), int(act),
                                     C.c_float(alpha), C.c_float(limit))
    return y


def forward_bf16(x_bits, logits, w13_bits, w2_bits, K, scoring="softmax", renormalize=True, n_group=1, topk_group=1,
                 routed_scale=1.0, bias=None, w13_bias=None, w2_bias=None, alpha=1.702, limit=7.0, f16=False,
                 first_expert=0):
    """Unquantized layer in the stage order of KunlunOps.fused_moe (ops/_kunlun_ops.py:412-637); with
    expert biases, its gpt-oss branch (:433-468): interleaved gate/up, swigluoai. first_expert: the weights are
    the experts [first_expert, first_expert + E) of those the logits run over (an expert-parallel share,
    :677-689): pairs routed elsewhere get no sorted row and add nothing."""
    E = w13_bits.shape[0]
    w, ids = _route(logits, K, scoring, renormalize, n_group, topk_group, routed_scale, bias)
    moe_index, src, _, lod = align(ids - np.int32(first_expert), E)
    if w13_bias is not None or w2_bias is not None:
        if f16:
            raise NotImplementedError("the expert-bias branch is restated for bf16 only")
        act = grouped_gemm_bf16_bias(x_bits, w13_bits, w13_bias, lod, act=2, row_src=src, src_div=K, alpha=alpha,
                                     limit=limit)
        down = grouped_gemm_bf16_bias(act, w2_bits, w2_bias, lod)
    else:
        act = grouped_gemm_bf16(x_bits, w13_bits, lod, act=1, row_src=src, src_div=K, f16=f16)
        down = grouped_gemm_bf16(act, w2_bits, lod, f16=f16)
    return combine(down, moe_index, w, f16=f16)


def forward_fp8(x_bits, logits, w13, w13_scale, w2, w2_scale, K, scoring="softmax", renormalize=True, n_group=1,
                topk_group=1, routed_scale=1.0, bias=None, shared=None, out_scale=1.0, f16=False):
    """fp8 block-scaled layer: same stage order as the int8 layer with the fp8 quantiser and GEMM; f16: x and out
    (and every 16-bit intermediate) hold IEEE half patterns."""
    E = w13.shape[0]
    M = x_bits.shape[0]
    w, ids = _route(logits, K, scoring, renormalize, n_group, topk_group, routed_scale, bias)
    moe_index, src, _, lod = align(ids, E)
    xq, xs = quant_fp8_group128(x_bits, f16=f16)
    act = grouped_gemm_fp8(xq, xs, w13, w13_scale, lod, act=1, row_src=src, src_div=K, f16=f16)
    aq, as_ = quant_fp8_group128(act, f16=f16)
    down = grouped_gemm_fp8(aq, as_, w2, w2_scale, lod, f16=f16)
    sh = None
    if shared is not None:
        ws13, ws13_scale, ws2, ws2_scale = shared
        dlod = np.array([0, M], np.int32)
        sact = grouped_gemm_fp8(xq, xs, ws13[None], ws13_scale[None], dlod, act=1, f16=f16)
        sq, ss = quant_fp8_group128(sact, f16=f16)
        sh = grouped_gemm_fp8(sq, ss, ws2[None], ws2_scale[None], dlod, f16=f16)
    return combine(down, moe_index, w, None, out_scale, sh, f16=f16)
