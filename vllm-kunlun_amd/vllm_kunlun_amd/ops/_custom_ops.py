"""torch.ops surface of the MoE path, backed by libkmoe.so.

Same operator names, argument names/order and out-parameter style as the
reference's shims in vllm_kunlun/ops/_custom_ops.py (each op cites its line
there); the body of every op is one call through the C ABI on the current HIP
stream. Nothing here computes with torch.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch.library import custom_op

from .. import _lib as L

_BF16 = torch.bfloat16


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def _act_bits(t: torch.Tensor, what: str) -> torch.Tensor:
    if t.dtype != _BF16:
        raise NotImplementedError(f"{what}: activations must be bfloat16, got {t.dtype}")
    return t


def _dt(t: torch.Tensor, what: str) -> int:
    """KMOE_DT_* of a bfloat16 or float16 activation tensor."""
    return L.act_dtype(t, what)


# --------------------------------------------------------------------- routing
@custom_op("_C::moe_softmax_topk", mutates_args=("normed_score", "topk_index"))
def moe_softmax_topk(x: torch.Tensor, normed_score: torch.Tensor, topk_index: torch.Tensor,
                     block_statistic: Optional[torch.Tensor], axis: int = -1, turn: bool = True) -> None:
    """softmax + top-K without renormalisation (reference: ops/_custom_ops.py:781-790)."""
    L.require_device(x, normed_score, topk_index)
    L.require_contig(x, normed_score, topk_index)
    _need(x.dtype == torch.float32 and normed_score.dtype == torch.float32 and topk_index.dtype == torch.int32,
          "moe_softmax_topk: x/normed_score must be float32 and topk_index int32")
    M, E = x.shape
    _need(tuple(normed_score.shape) == tuple(topk_index.shape) and normed_score.shape[0] == M,
          "moe_softmax_topk: output shapes must be [M, K]")
    L.check(L.lib.kmoe_softmax_topk(L.ptr(x), M, E, normed_score.shape[1], 0, L.ptr(normed_score),
                                    L.ptr(topk_index), L.stream()))


@custom_op("_C::moe_softmax_topk_norm", mutates_args=("normed_score", "topk_index"))
def moe_softmax_topk_norm(x: torch.Tensor, normed_score: torch.Tensor, topk_index: torch.Tensor,
                          block_statistic: Optional[torch.Tensor], stable: bool = True) -> None:
    """softmax + top-K + renormalise (reference: ops/_custom_ops.py:1084-1094).
    `stable` is accepted for signature parity; ties always go to the lower expert id."""
    L.require_device(x, normed_score, topk_index)
    L.require_contig(x, normed_score, topk_index)
    _need(x.dtype == torch.float32 and normed_score.dtype == torch.float32 and topk_index.dtype == torch.int32,
          "moe_softmax_topk_norm: x/normed_score must be float32 and topk_index int32")
    M, E = x.shape
    _need(tuple(normed_score.shape) == tuple(topk_index.shape) and normed_score.shape[0] == M,
          "moe_softmax_topk_norm: output shapes must be [M, K]")
    L.check(L.lib.kmoe_softmax_topk(L.ptr(x), M, E, normed_score.shape[1], 1, L.ptr(normed_score),
                                    L.ptr(topk_index), L.stream()))


@custom_op("_C::moe_sigmoid_group_topk_norm", mutates_args=("topk_index", "norm_score", "block_static"))
def moe_sigmoid_group_topk_norm(x: torch.Tensor, topk_index: torch.Tensor, norm_score: torch.Tensor,
                                block_static: Optional[torch.Tensor], bias: Optional[torch.Tensor], scale: float,
                                n_group: Optional[int], topk_group: Optional[int]) -> None:
    """DeepSeek-V3 grouped top-K with correction bias (reference: ops/_custom_ops.py:1351-1371).
    When block_static [B, E] is given it also receives the per-block histogram of the chosen ids."""
    L.require_device(x, topk_index, norm_score, bias, block_static)
    L.require_contig(x, topk_index, norm_score, bias, block_static)
    _need(x.dtype == torch.float32 and norm_score.dtype == torch.float32 and topk_index.dtype == torch.int32,
          "moe_sigmoid_group_topk_norm: x/norm_score must be float32 and topk_index int32")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == x.shape[1]),
          "moe_sigmoid_group_topk_norm: bias must be float32 [E]")
    M, E = x.shape
    K = topk_index.shape[1]
    L.check(L.lib.kmoe_sigmoid_group_topk_norm(L.ptr(x), L.ptr(bias), M, E, K, int(n_group or 1), int(topk_group or 1),
                                               float(scale), L.ptr(norm_score), L.ptr(topk_index), L.stream()))
    if block_static is not None and block_static.numel() > 0:
        _need(block_static.dtype == torch.int32 and block_static.dim() == 2 and block_static.shape[1] == E,
              "moe_sigmoid_group_topk_norm: block_static must be int32 [B, E]")
        L.check(L.lib.kmoe_block_statistic(L.ptr(topk_index), M * K, E, block_static.shape[0], L.ptr(block_static),
                                           L.stream()))


@custom_op("_moe_C::topk_softmax", mutates_args=("topk_weights", "topk_ids", "token_expert_indices"))
def topk_softmax(topk_weights: torch.Tensor, topk_ids: torch.Tensor, token_expert_indices: torch.Tensor,
                 gating_output: torch.Tensor, renormalize: bool = False,
                 e_score_correction_bias: Optional[torch.Tensor] = None) -> None:
    """Upstream's non-monolithic routing op; an empty stub in the reference
    (ops/_custom_ops.py:8-17, prototype csrc/xops.h:162-166), real here."""
    if e_score_correction_bias is not None:
        raise NotImplementedError("topk_softmax: correction bias belongs to moe_sigmoid_group_topk_norm")
    L.require_device(topk_weights, topk_ids, gating_output)
    L.require_contig(topk_weights, topk_ids, gating_output)
    _need(gating_output.dtype == torch.float32 and topk_weights.dtype == torch.float32
          and topk_ids.dtype == torch.int32, "topk_softmax: float32 scores/weights and int32 ids expected")
    M, E = gating_output.shape
    K = topk_ids.shape[1]
    L.check(L.lib.kmoe_softmax_topk(L.ptr(gating_output), M, E, K, int(renormalize), L.ptr(topk_weights),
                                    L.ptr(topk_ids), L.stream()))
    if token_expert_indices.numel() == M * K:  # upstream convention: k * M + m
        idx = torch.arange(K, device=topk_ids.device, dtype=torch.int32)[None, :] * M + \
            torch.arange(M, device=topk_ids.device, dtype=torch.int32)[:, None]
        token_expert_indices.copy_(idx)


# ----------------------------------------------------------------------- align
@custom_op("_C::gen_block_statistic", mutates_args=("block_statistic",))
def gen_block_statistic(topk_ids: torch.Tensor, block_statistic: torch.Tensor) -> None:
    """Per-block expert histogram [B, E] (reference: ops/_custom_ops.py:1123-1125)."""
    L.require_device(topk_ids, block_statistic)
    L.require_contig(topk_ids, block_statistic)
    _need(topk_ids.dtype == torch.int32 and block_statistic.dtype == torch.int32 and block_statistic.dim() == 2,
          "gen_block_statistic: int32 ids and int32 [B, E] histogram expected")
    B, E = block_statistic.shape
    L.check(L.lib.kmoe_block_statistic(L.ptr(topk_ids), topk_ids.numel(), E, B, L.ptr(block_statistic), L.stream()))


def _align(topk_index: torch.Tensor, E: int, moe_index: torch.Tensor, sorted_src: torch.Tensor,
           expert_m: Optional[torch.Tensor], lod: torch.Tensor) -> None:
    P = topk_index.numel()
    ws_bytes = L.lib.kmoe_align_workspace_bytes(P, E)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=topk_index.device)
    L.check(L.lib.kmoe_align(L.ptr(topk_index), P, E, L.ptr(moe_index), L.ptr(sorted_src), L.ptr(expert_m),
                             L.ptr(lod), L.ptr(ws), ws_bytes, L.stream()))


@custom_op("_C::moe_pre_sorted", mutates_args=("moe_expand", "moe_index", "expert_m", "sorted_tokens_num_lod"))
def moe_pre_sorted(x: torch.Tensor, topk_index: torch.Tensor, block_statistic: Optional[torch.Tensor],
                   moe_expand: torch.Tensor, moe_index: torch.Tensor, expert_m: torch.Tensor,
                   sorted_tokens_num_lod: torch.Tensor, index_have_neg: bool = False) -> None:
    """Stable sort of routed pairs by expert + gather of their activation rows
    (reference: ops/_custom_ops.py:1144-1163). block_statistic is not needed: the
    histograms are rebuilt in LDS."""
    L.require_device(x, topk_index, moe_expand, moe_index, expert_m, sorted_tokens_num_lod)
    L.require_contig(x, topk_index, moe_expand, moe_index, expert_m, sorted_tokens_num_lod)
    _need(topk_index.dtype == torch.int32 and moe_index.dtype == torch.int32 and expert_m.dtype == torch.int32
          and sorted_tokens_num_lod.dtype == torch.int32, "moe_pre_sorted: index tensors must be int32")
    _need(x.element_size() == 2 and moe_expand.dtype == x.dtype, "moe_pre_sorted: x/moe_expand must be 16-bit and alike")
    M, H = x.shape
    K = topk_index.shape[1]
    E = expert_m.numel()
    P = M * K
    _need(moe_index.numel() == P and sorted_tokens_num_lod.numel() == E + 1 and moe_expand.numel() == P * H,
          "moe_pre_sorted: output shapes do not match M, K, E, H")
    sorted_src = torch.empty(P, dtype=torch.int32, device=x.device)
    _align(topk_index, E, moe_index, sorted_src, expert_m, sorted_tokens_num_lod)
    L.check(L.lib.kmoe_gather_rows(L.ptr(x), H, L.ptr(sorted_src), P, K, H, L.ptr(moe_expand), H, L.stream()))


@custom_op("xspeedgate_ops::moe_pre_small", mutates_args=())
def moe_pre_small(topk_ids: torch.Tensor, global_num_experts: int, index_have_neg: bool, sort_mode: bool,
                  x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Small-P variant of moe_pre_sorted that allocates its outputs
    (reference call: compressed_tensors_moe.py:199-207). Returns
    (sorted_tokens_idx [P], sorted_tokens_num_lod [E+1], moe_expand [P, H])."""
    L.require_device(topk_ids, x)
    L.require_contig(topk_ids, x)
    M, H = x.shape
    P = topk_ids.numel()
    E = int(global_num_experts)
    dev = x.device
    moe_index = torch.empty(P, dtype=torch.int32, device=dev)
    sorted_src = torch.empty(P, dtype=torch.int32, device=dev)
    lod = torch.empty(E + 1, dtype=torch.int32, device=dev)
    moe_expand = torch.empty(P, H, dtype=x.dtype, device=dev)
    _align(topk_ids, E, moe_index, sorted_src, None, lod)
    L.check(L.lib.kmoe_gather_rows(L.ptr(x), H, L.ptr(sorted_src), P, topk_ids.shape[1], H, L.ptr(moe_expand), H,
                                   L.stream()))
    return moe_index, lod, moe_expand


# ----------------------------------------------------------------------- quant
@custom_op("_C::quant2d", mutates_args=("x_q", "max"))
def quant2d(x: torch.Tensor, x_q: torch.Tensor, max: torch.Tensor, force_sdnn: bool = False) -> None:
    """Per-row dynamic int8; `max` receives the row ABSMAX (reference: ops/_custom_ops.py:1912-1924)."""
    L.require_device(x, x_q, max)
    L.require_contig(x, x_q, max)
    dt = _dt(x, "quant2d")
    _need(x_q.dtype == torch.int8 and max.dtype == torch.float32, "quant2d: x_q must be int8 and max float32")
    C = x.shape[-1]
    R = x.numel() // C
    _need(x_q.numel() == x.numel() and max.numel() == R, "quant2d: x_q/max shapes do not match x")
    L.check(L.lib.kmoe_quant_i8_rows_dt(L.ptr(x), C, R, C, L.ptr(x_q), C, L.ptr(max), dt, L.stream()))


@custom_op("_C::scaled_int8_quant", mutates_args=())
def scaled_int8_quant(x: torch.Tensor, scale: Optional[torch.Tensor], azp: Optional[torch.Tensor] = None,
                      symmetric: bool = True) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, bool]:
    """int8 quantisation of activations (reference: ops/_custom_ops.py:1633-1657): returns (codes, scale, azp,
    static). Dynamic symmetric (scale None, symmetric): per token, and the returned `scale` holds the row MAX, as in
    the reference (quant2d). Static (scale given: one f32 for the tensor, optionally a zero point azp): codes =
    sat8(rint(x / scale) + azp). Dynamic asymmetric (scale None, not symmetric): per token scale = (max - min) / 255
    and zero point rint(-128 - min / scale). Where the reference returns azp = None this returns an empty tensor
    (operator schemas cannot return None)."""
    L.require_device(x, scale, azp)
    xc = x.contiguous()
    rows, cols = xc.numel() // xc.shape[-1], xc.shape[-1]
    x_q = torch.empty_like(xc, dtype=torch.int8)
    none = torch.empty(0, dtype=torch.int32, device=x.device)
    dt = L.act_dtype(xc, "scaled_int8_quant")
    if scale is not None:  # static
        _need(scale.numel() == 1 and scale.dtype == torch.float32, "scaled_int8_quant: the static scale is one float32")
        _need(azp is None or (azp.numel() == 1 and azp.dtype == torch.int32),
              "scaled_int8_quant: the static zero point is one int32")
        if rows:
            L.check(L.lib.kmoe_quant_i8_static(L.ptr(xc), cols, rows, cols, L.ptr(scale), L.ptr(azp), L.ptr(x_q), cols, dt,
                                               L.stream()))
        # (copies: an operator's results may not alias its arguments)
        return x_q, scale.clone(), none if azp is None else azp.clone(), True
    if symmetric:
        mx = torch.empty((rows, 1), device=x.device, dtype=torch.float32)
        quant2d(xc, x_q, mx, True)
        return x_q, mx, none, False
    s = torch.empty((rows, 1), device=x.device, dtype=torch.float32)
    z = torch.empty((rows, 1), device=x.device, dtype=torch.int32)
    if rows:
        L.check(L.lib.kmoe_quant_i8_rows_azp(L.ptr(xc), cols, rows, cols, L.ptr(x_q), cols, L.ptr(s), L.ptr(z), dt,
                                             L.stream()))
    return x_q, s, z, False


# ------------------------------------------------------------------------ GEMM
def _gemm_i8(a, a_max, w, w_max, lod, y2d, ldy, act, rows, row_src=None, src_div=1, acc_out=None, variant=0):
    from .._plan import weight_layout
    E, n, k = w.shape
    args = L.GemmI8Args()
    args.a = a.data_ptr()
    args.lda = a.stride(0)
    args.a_max = a_max.data_ptr()
    args.row_src = 0 if row_src is None else row_src.data_ptr()
    args.src_div = src_div
    args.w = w.data_ptr()
    args.w_max = w_max.data_ptr()
    args.lod = lod.data_ptr()
    args.E, args.n, args.k, args.rows = E, n, k, rows
    args.y = y2d.data_ptr()
    args.ldy = ldy
    args.acc_out = 0 if acc_out is None else acc_out.data_ptr()
    args.act = act
    args.variant = variant
    args.w_layout = weight_layout(w)
    args.act_dtype = L.act_dtype(y2d, "int8 GEMM output")
    L.check(L.lib.kmoe_grouped_gemm_i8(args, L.stream()))


def _moe_fc_fp8(x, weight, lod, y, act, x_scale, w_scale, scale_n, scale_k) -> None:
    """moe_fc with scale_n / scale_k (reference: ops/_custom_ops.py:1218-1221 merely passes them on): block-scaled
    fp8-e4m3fn operands, one weight scale per scale_n x scale_k block, one activation scale per row and scale_k
    columns. 128 x 128 blocks (the DeepSeek-V3 recipe) are what the kernels serve."""
    from .._plan import weight_layout
    if (scale_n, scale_k) != (128, 128):
        raise NotImplementedError(f"moe_fc: block scales of {scale_n} x {scale_k} are not served (128 x 128 only)")
    f8 = (torch.float8_e4m3fn, torch.uint8)
    _need(x.dtype in f8 and weight.dtype in f8, "moe_fc: block-scaled operands must be float8_e4m3fn (or their bytes)")
    _need(y.dtype in (_BF16, torch.float16), "moe_fc: the block-scaled GEMM writes bfloat16 or float16")
    E, n, k = weight.shape
    rows = x.numel() // k
    _need(x_scale is not None and w_scale is not None and x_scale.dtype == torch.float32
          and w_scale.dtype == torch.float32, "moe_fc: block-scaled operands need float32 scales")
    _need(x_scale.numel() == rows * (k // 128) and w_scale.numel() == E * (n // 128) * (k // 128),
          "moe_fc: scales must be [P, k/128] and [E, n/128, k/128]")
    n_out = n // 2 if act else n
    _need(y.numel() in (rows * n_out, rows * n) and lod.numel() == E + 1, "moe_fc: x/y/lod shapes do not match weight")
    g = L.GemmFp8Args()
    g.a, g.lda, g.a_scale, g.src_div = x.data_ptr(), k, x_scale.data_ptr(), 1
    g.w, g.w_scale, g.lod = weight.data_ptr(), w_scale.data_ptr(), lod.data_ptr()
    g.E, g.n, g.k, g.rows = E, n, k, rows
    g.y, g.ldy = y.data_ptr(), y.numel() // max(rows, 1) if rows else n_out
    g.act = L.KMOE_ACT_SWIGLU if act else L.KMOE_ACT_NONE
    g.w_layout = weight_layout(weight)
    g.act_dtype = L.act_dtype(y)
    L.check(L.lib.kmoe_grouped_gemm_fp8_block(g, L.stream()))


def _moe_fc_w4(x, weight, lod, y, act, w_scale, group_size) -> None:
    """moe_fc with use_pack_int4: bfloat16 (or float16) activations against packed 4-bit weights [E, n, k/2] (two
    codes per byte, low nibble first, code - 8; re-tiled at load time) with group scales [E, n, k/group] in the
    activations' dtype; scale_k carries the group size (0: one scale per output channel)."""
    from .._plan import scale_layout, weight_layout
    _need(x.dtype in (_BF16, torch.float16) and y.dtype == x.dtype and weight.dtype == torch.uint8,
          "moe_fc: packed 4-bit weights are uint8 and go with bfloat16 or float16 activations")
    E, n, half_k = weight.shape
    k = 2 * half_k
    rows = x.numel() // k
    gs = group_size or k
    _need(w_scale is not None and w_scale.dtype == x.dtype and w_scale.numel() == E * n * (k // gs),
          "moe_fc: packed 4-bit weights need scales [E, n, k/group] in the activations' dtype")
    if weight_layout(weight) != L.KMOE_W_TILED:
        raise NotImplementedError("moe_fc: packed 4-bit weights must be re-tiled (tile_int8_weights_) first")
    n_out = n // 2 if act else n
    g = L.GemmW4Args()
    g.a, g.lda, g.src_div = x.data_ptr(), k, 1
    g.w, g.w_scale, g.group_size, g.lod = weight.data_ptr(), w_scale.data_ptr(), gs, lod.data_ptr()
    g.E, g.n, g.k, g.rows = E, n, k, rows
    g.y, g.ldy = y.data_ptr(), y.numel() // max(rows, 1) if rows else n_out
    g.act = L.KMOE_ACT_SWIGLU if act else L.KMOE_ACT_NONE
    g.w_layout = L.KMOE_W_TILED
    g.act_dtype = L.act_dtype(x)
    g.scale_layout = scale_layout(w_scale)  # re-arranged at load time (tile_w4_scales_), or as the checkpoint holds them
    L.check(L.lib.kmoe_grouped_gemm_w4a16(g, L.stream()))


@custom_op("_C::moe_fc", mutates_args=("y",))
def moe_fc(x: torch.Tensor, weight: torch.Tensor, sorted_tokens_num_lod: torch.Tensor,
           sorted_tokens_idx: torch.Tensor, moe_topk: int, y: torch.Tensor, act: Optional[str] = None,
           x_perchannel_max: Optional[torch.Tensor] = None, w_perchannel_max: Optional[torch.Tensor] = None,
           topk_ids: Optional[torch.Tensor] = None, topk_w: Optional[torch.Tensor] = None,
           bias: Optional[torch.Tensor] = None, tgemm_type: Optional[str] = None,
           tweight_type: Optional[str] = None, scale_n: Optional[int] = 0, scale_k: Optional[int] = 0,
           use_pack_int4: Optional[bool] = False, sort_mode: Optional[bool] = True) -> None:
    """Grouped GEMM over sorted rows (reference: ops/_custom_ops.py:1204-1244).
    x [P, k] holds the rows in sorted order; rows [lod[e], lod[e+1]) meet weight[e] [n, k].
    int8 x/weight with x_perchannel_max [P,1] and w_perchannel_max [E,n,1] give the
    W8A8 path; act="SWISH_GLU" writes silu(gate)*up into the first n/2 columns of y."""
    L.require_device(x, weight, sorted_tokens_num_lod, y, x_perchannel_max, w_perchannel_max)
    L.require_contig(x, weight, sorted_tokens_num_lod, y, x_perchannel_max, w_perchannel_max)
    if bias is not None or topk_w is not None:
        raise NotImplementedError("moe_fc: bias / topk_w are not on this path")
    _need(act in (None, "SWISH_GLU"), f"moe_fc: act={act!r} unknown")
    _dt(y, "moe_fc")
    if use_pack_int4:
        return _moe_fc_w4(x, weight, sorted_tokens_num_lod, y, act, w_perchannel_max, int(scale_k or 0))
    if scale_n or scale_k:
        return _moe_fc_fp8(x, weight, sorted_tokens_num_lod, y, act, x_perchannel_max, w_perchannel_max,
                           int(scale_n or 0), int(scale_k or 0))
    E, n, k = weight.shape
    rows = x.numel() // k
    _need(x.shape[-1] == k and y.numel() == rows * n and sorted_tokens_num_lod.numel() == E + 1,
          "moe_fc: x/y/lod shapes do not match weight")
    if x.dtype == torch.int8:
        _need(weight.dtype == torch.int8 and x_perchannel_max is not None and w_perchannel_max is not None,
              "moe_fc: int8 x needs int8 weight and both per-channel max tensors")
        _need(x_perchannel_max.numel() == rows and w_perchannel_max.numel() == E * n,
              "moe_fc: per-channel max shapes must be [P,1] and [E,n,1]")
        _gemm_i8(x.view(rows, k), x_perchannel_max, weight, w_perchannel_max, sorted_tokens_num_lod,
                 y, n, L.KMOE_ACT_SWIGLU if act else L.KMOE_ACT_NONE, rows)
    elif x.dtype in (_BF16, torch.float16):
        _need(weight.dtype == x.dtype and y.dtype == x.dtype, "moe_fc: unquantized x needs weight and y of its dtype")
        g = L.GemmBf16Args()
        g.act_dtype = L.act_dtype(x)
        g.a, g.lda, g.src_div = x.data_ptr(), k, 1
        g.w, g.lod = weight.data_ptr(), sorted_tokens_num_lod.data_ptr()
        g.E, g.n, g.k, g.rows = E, n, k, rows
        g.y, g.ldy = y.data_ptr(), n
        g.act = L.KMOE_ACT_SWIGLU if act else L.KMOE_ACT_NONE
        from .._plan import weight_layout
        g.w_layout = weight_layout(weight)
        L.check(L.lib.kmoe_grouped_gemm_bf16(g, L.stream()))
    else:
        raise NotImplementedError(f"moe_fc: x dtype {x.dtype} is outside this build's path (int8, bfloat16 or float16)")


_DENSE_LOD: dict = {}


def _dense_lod(device: torch.device, rows: int) -> torch.Tensor:
    """The row range {0, rows} of a dense GEMM's single expert, on the device; made once per
    (device, rows) so that a replayed or captured call copies nothing from the host."""
    key = (device.type, device.index if device.index is not None else torch.cuda.current_device(), rows)
    lod = _DENSE_LOD.get(key)
    if lod is None:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError(f"matmul: run one call with {rows} rows before capturing (its row range is "
                               "uploaded once per size)")
        lod = torch.tensor([0, rows], dtype=torch.int32).to(device)
        _DENSE_LOD[key] = lod
    return lod


@custom_op("_C::matmul", mutates_args=())
def matmul(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, x_trans: bool = False, w_trans: bool = True,
           alpha: float = 1.0, beta: float = 0.0, bias: Optional[torch.Tensor] = None,
           x_max: Optional[torch.Tensor] = None, w_max: Optional[torch.Tensor] = None,
           x_pc_max: Optional[torch.Tensor] = None, w_pc_max: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Dense W8A8 linear: x int8 [M,k] with per-row max, w int8 [n,k] with per-channel
    max -> out [M,n] (reference: ops/_custom_ops.py:1811-1845; caller
    quantization/kernels/scale_mm.py:83-90). One-expert case of the grouped GEMM; with a bias (f32 [n]) its int32
    sums are rescaled and the bias added in a second pass (kmoe_scaled_mm_azp_epilogue without a zero point)."""
    if x.dtype != torch.int8 or w.dtype != torch.int8 or x_pc_max is None or w_pc_max is None:
        raise NotImplementedError("matmul: only the int8 path with x_pc_max / w_pc_max is implemented")
    if x_trans or not w_trans or alpha != 1.0 or beta != 0.0:
        raise NotImplementedError("matmul: x_trans / w_trans=False / alpha / beta are not on this path")
    if out_dtype not in (_BF16, torch.float16):
        raise NotImplementedError(f"matmul: out_dtype {out_dtype} is not implemented")
    L.require_device(x, w, x_pc_max, w_pc_max)
    from .._plan import is_tiled
    # weights re-tiled at load time come in as a view of their memory (e.g. layer.weight.t()): a copy made by
    # .contiguous() would shuffle tiled bytes, so such a weight must already be the contiguous [n, k] tensor
    # (_gemm_i8 refuses any other view of tiled memory)
    xc, wc = x.contiguous(), (w if is_tiled(w) else w.contiguous())
    M, k = xc.shape
    n = wc.shape[0]
    out = torch.empty((M, n), dtype=out_dtype, device=x.device)
    if x_pc_max.numel() == 1 and M != 1:  # one max for the tensor (static quantisation): every row's
        x_pc_max = x_pc_max.reshape(1).expand(M)
    acc = None
    if bias is not None and M:  # the GEMM leaves its int32 sums as well; the epilogue below rescales them and adds
        _need(bias.dtype == torch.float32 and bias.numel() == n, "matmul: bias is f32 [n]")
        L.require_device(bias)
        acc = torch.empty((M, n), dtype=torch.int32, device=x.device)
    x_max, w_max = x_pc_max.contiguous(), w_pc_max.contiguous()
    _gemm_i8(xc, x_max, wc.unsqueeze(0), w_max, _dense_lod(x.device, M), out, n, L.KMOE_ACT_NONE, M, acc_out=acc)
    if acc is not None:
        L.check(L.lib.kmoe_scaled_mm_azp_epilogue(L.ptr(acc), n, M, n, L.ptr(x_max), 1, L.ptr(w_max), 1, None, None,
                                                  L.ptr(bias.contiguous()), L.ptr(out), n, L.act_dtype(out), L.stream()))
    return out


@custom_op("_C::cutlass_scaled_mm_azp", mutates_args=())
def cutlass_scaled_mm_azp(a: torch.Tensor, b: torch.Tensor, scale_a: torch.Tensor, scale_b: torch.Tensor,
                          out_dtype: torch.dtype, azp_adj: torch.Tensor, azp: Optional[torch.Tensor] = None,
                          bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Dense W8A8 linear with asymmetric activations (reference: ops/_custom_ops.py:1756-1771; caller
    quantization/kernels/scale_mm.py:70-82): a int8 [M,k] (codes with a zero point), b int8 [k,n] (the transpose
    view of the [n,k] weight), scale_a f32 [M,1] or [1], scale_b f32 [1,n] or [1], azp_adj int32 [1,n] (sums of
    the weight codes over k, times the zero point for a static scheme), azp int32 [M,1] or None, bias f32 [n]:
    out = scale_a * scale_b * (a @ b - azp * azp_adj) + bias. The int8 GEMM leaves its int32 accumulators
    (acc_out of kmoe_grouped_gemm_i8); kmoe_scaled_mm_azp_epilogue finishes them."""
    if a.dtype != torch.int8 or b.dtype != torch.int8 or a.dim() != 2 or b.dim() != 2:
        raise NotImplementedError("cutlass_scaled_mm_azp: int8 a [M,k] and b [k,n] only")
    if out_dtype not in (_BF16, torch.float16):
        raise NotImplementedError(f"cutlass_scaled_mm_azp: out_dtype {out_dtype} is not implemented")
    L.require_device(a, b, scale_a, scale_b, azp_adj, azp, bias)
    from .._plan import is_tiled
    w = b.t()  # the [n, k] weight; re-tiled memory must come as the transpose view of the tensor that was tiled
    if not is_tiled(w):
        w = w.contiguous()
    ac = a.contiguous()
    M, k = ac.shape
    n = w.shape[0]
    _need(w.shape[1] == k and azp_adj.numel() == n and azp_adj.dtype == torch.int32,
          "cutlass_scaled_mm_azp: b must be [k,n] and azp_adj int32 with n entries")
    _need(scale_a.dtype == torch.float32 and scale_a.numel() in (1, M) and scale_b.dtype == torch.float32
          and scale_b.numel() in (1, n), "cutlass_scaled_mm_azp: f32 scales, one per row / channel or one per tensor")
    _need(azp is None or (azp.dtype == torch.int32 and azp.numel() == M), "cutlass_scaled_mm_azp: azp is int32 [M,1]")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n), "cutlass_scaled_mm_azp: bias is f32 [n]")
    out = torch.empty((M, n), dtype=out_dtype, device=a.device)
    if M == 0:
        return out
    acc = torch.empty((M, n), dtype=torch.int32, device=a.device)
    ones_m, ones_n = _ones(a.device, M), _ones(a.device, n)  # the GEMM's own rescaling is not used
    _gemm_i8(ac, ones_m, w.unsqueeze(0), ones_n, _dense_lod(a.device, M), out, n, L.KMOE_ACT_NONE, M, acc_out=acc)
    L.check(L.lib.kmoe_scaled_mm_azp_epilogue(
        L.ptr(acc), n, M, n, L.ptr(scale_a.contiguous()), int(scale_a.numel() == M),
        L.ptr(scale_b.contiguous()), int(scale_b.numel() == n), L.ptr(azp_adj.contiguous()),
        L.ptr(None if azp is None else azp.contiguous()), L.ptr(None if bias is None else bias.contiguous()), L.ptr(out),
        n, L.act_dtype(out), L.stream()))
    return out


_ONES: dict = {}


def _ones(device: torch.device, count: int) -> torch.Tensor:
    key = (device.type, device.index if device.index is not None else torch.cuda.current_device(), count)
    t = _ONES.get(key)
    if t is None:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("cutlass_scaled_mm_azp: run one call of this size before capturing")
        t = _ONES[key] = torch.ones(count, dtype=torch.float32, device=device)
    return t


# ---------------------------------------------------------------- elementwise
@custom_op("_C::silu_and_mul", mutates_args=("out",))
def silu_and_mul(out: torch.Tensor, x: torch.Tensor, axis: int = -1, turn: bool = True) -> None:
    """out = silu(x[..., :d]) * x[..., d:] (reference: ops/_custom_ops.py:699-706)."""
    L.require_device(out, x)
    L.require_contig(out, x)
    dt = _dt(x, "silu_and_mul")
    _need(out.dtype == x.dtype, "silu_and_mul: out and x must share a dtype")
    two_i = x.shape[-1]
    R = x.numel() // two_i
    _need(two_i % 2 == 0 and out.numel() == R * (two_i // 2), "silu_and_mul: out must be [..., d] for x [..., 2d]")
    L.check(L.lib.kmoe_silu_and_mul_dt(L.ptr(x), two_i, R, two_i // 2, L.ptr(out), two_i // 2, dt, L.stream()))


@custom_op("_C::moe_post", mutates_args=("y",))
def moe_post(x: torch.Tensor, moe_index: torch.Tensor, normed_scale: torch.Tensor, dequant_scale: torch.Tensor,
             y: torch.Tensor) -> None:
    """y[m] = sum_k normed_scale[m,k] * dequant_scale[m,k] * x[moe_index[m,k]]
    (reference: ops/_custom_ops.py:1316-1324)."""
    L.require_device(x, moe_index, normed_scale, dequant_scale, y)
    L.require_contig(x, moe_index, normed_scale, dequant_scale, y)
    dt = _dt(x, "moe_post")
    _need(y.dtype == x.dtype and moe_index.dtype == torch.int32 and normed_scale.dtype == torch.float32
          and dequant_scale.dtype == torch.float32, "moe_post: dtypes must be (x, int32, float32, float32, x)")
    M, H = y.shape
    K = moe_index.numel() // M
    _need(x.numel() == M * K * H and normed_scale.numel() == M * K and dequant_scale.numel() == M * K,
          "moe_post: shapes must be x [M,K,H], index/scales [M,K], y [M,H]")
    L.check(L.lib.kmoe_combine_dt(L.ptr(x), H, L.ptr(moe_index), L.ptr(normed_scale), L.ptr(dequant_scale), M, K, H,
                                  1.0, None, 0, 1.0, L.ptr(y), H, dt, L.stream()))


# Fake (meta) implementations so the ops can be traced, as the reference registers for each op.
@custom_op("_C::swigluoai_and_mul", mutates_args=())
def swigluoai_and_mul(x: torch.Tensor, alpha: float = 1.702, limit: float = 7.0, axis: int = -1,
                      turn: bool = True) -> torch.Tensor:
    """gate = x[..., ::2], up = x[..., 1::2]; (up.clamp(-limit, limit) + 1) * g * sigmoid(alpha * g) with
    g = gate.clamp(max=limit) (reference: ops/_custom_ops.py:728-742)."""
    _need(axis in (-1, x.dim() - 1), "swigluoai_and_mul: only the last axis")
    bits_in = _act_bits(x, "swigluoai_and_mul")
    x2 = bits_in.reshape(-1, x.shape[-1])
    _need(x2.shape[1] % 8 == 0, "swigluoai_and_mul: the last dimension must be a multiple of 8")
    L.require_device(x2)
    out = torch.empty((*x.shape[:-1], x.shape[-1] // 2), dtype=x.dtype, device=x.device)
    L.check(L.lib.kmoe_swigluoai_and_mul(L.ptr(x2), x2.shape[1], x2.shape[0], x2.shape[1] // 2, float(alpha),
                                         float(limit), L.ptr(out), x2.shape[1] // 2, L.stream()))
    return out


@swigluoai_and_mul.register_fake
def _fake_swigluoai_and_mul(x, alpha=1.702, limit=7.0, axis=-1, turn=True):
    return x.new_empty((*x.shape[:-1], x.shape[-1] // 2))


@custom_op("_C::router_gemm_bf16_fp32", mutates_args=())
def router_gemm_bf16_fp32(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """bf16 [M,H] x bf16 [E,H]^T -> f32 [M,E] router logits (reference: ops.router_gemm_bf16_fp32,
    ops/fused_moe/router/gate_linear.py:105-108)."""
    _need(x.dtype in (torch.bfloat16, torch.float16) and weight.dtype == x.dtype,
          "router_gemm_bf16_fp32: bfloat16 (or float16) inputs of one dtype")
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1], "router_gemm_bf16_fp32: shapes")
    L.require_device(x, weight)
    x, weight = x.contiguous(), weight.contiguous()
    M, H = x.shape
    E = weight.shape[0]
    out = torch.empty((M, E), dtype=torch.float32, device=x.device)
    nbytes = L.lib.kmoe_router_gemm_workspace_bytes(M, H, E)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    L.check(L.lib.kmoe_router_gemm(L.ptr(x), H, L.ptr(weight), M, H, E, L.ptr(out), E, L.ptr(ws), nbytes,
                                   L.act_dtype(x, "router_gemm"), L.stream()))
    return out


@router_gemm_bf16_fp32.register_fake
def _fake_router_gemm(x, weight):
    return x.new_empty((x.shape[0], weight.shape[0]), dtype=torch.float32)


def _none(*args, **kwargs):
    return None


for _op in (moe_softmax_topk, moe_softmax_topk_norm, moe_sigmoid_group_topk_norm, topk_softmax, gen_block_statistic,
            moe_pre_sorted, quant2d, moe_fc, silu_and_mul, moe_post):
    _op.register_fake(_none)


@moe_pre_small.register_fake
def _fake_moe_pre_small(topk_ids, global_num_experts, index_have_neg, sort_mode, x):
    P = topk_ids.numel()
    return (torch.empty(P, dtype=torch.int32, device=x.device),
            torch.empty(global_num_experts + 1, dtype=torch.int32, device=x.device),
            torch.empty(P, x.shape[1], dtype=x.dtype, device=x.device))


@scaled_int8_quant.register_fake
def _fake_scaled_int8_quant(x, scale, azp=None, symmetric=True):
    rows = x.numel() // x.shape[-1]
    none = torch.empty(0, dtype=torch.int32, device=x.device)
    if scale is not None:
        return torch.empty_like(x, dtype=torch.int8), torch.empty_like(scale), none if azp is None else torch.empty_like(azp), True
    return (torch.empty_like(x, dtype=torch.int8), torch.empty((rows, 1), device=x.device, dtype=torch.float32),
            none if symmetric else torch.empty((rows, 1), device=x.device, dtype=torch.int32), False)


@cutlass_scaled_mm_azp.register_fake
def _fake_cutlass_scaled_mm_azp(a, b, scale_a, scale_b, out_dtype, azp_adj, azp=None, bias=None):
    return torch.empty((a.shape[0], b.shape[1]), dtype=out_dtype, device=a.device)


@matmul.register_fake
def _fake_matmul(x, w, out_dtype, x_trans=False, w_trans=True, alpha=1.0, beta=0.0, bias=None, x_max=None,
                 w_max=None, x_pc_max=None, w_pc_max=None):
    return torch.empty((x.shape[0], w.shape[0] if w_trans else w.shape[1]), dtype=out_dtype, device=x.device)
