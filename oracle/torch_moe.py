"""torch-CPU restatement of the reference's own torch MoE computation — TEST INFRASTRUCTURE.

This is the path bench.py times as `cpu_baseline` ("port") and the second,
independently written oracle the tests hold the C restatement against. It
follows, with ordinary torch ops and no custom kernels:

  * the per-expert masked loop of KunlunOps.fused_moe_ep
    (vllm_kunlun/ops/_kunlun_ops.py:655-696): repeat_interleave of the tokens,
    a boolean mask per expert over the flat ids, gate_up matmul, silu_and_mul,
    down matmul, masked scatter, weighted sum over the K slots;
  * driven, for W8A8, by the stage order and dtypes of
    KunlunCompressedTensorsW8A8Int8MoEMethod.apply_monolithic
    (vllm_kunlun/quantization/compressed_tensors/compressed_tensors_moe.py:151-291):
    f32 routing, quant2d (max = absmax), int8 x int8 -> int32, dequant by
    x_max * w_max / 127^2 into bf16, silu_and_mul in bf16, quant2d again, down
    GEMM, moe_post with f32 weights;
  * routing variants of compressed_tensors_moe.py:152-170.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import it.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


# ------------------------------------------------------------------ routing
def softmax_topk(logits: torch.Tensor, K: int, renorm: bool):
    """moe_softmax_topk(_norm): softmax over experts, top-K, optional renormalise."""
    p = torch.softmax(logits.float(), dim=-1)
    w, ids = torch.topk(p, K, dim=-1)
    if renorm:
        w = w / w.sum(dim=-1, keepdim=True)
    return w, ids.to(torch.int32)


def sigmoid_group_topk_norm(logits, bias, K, n_group, topk_group, scale):
    """moe_sigmoid_group_topk_norm: DeepSeek-V3 grouped top-k with correction bias."""
    s = torch.sigmoid(logits.float())
    c = s if bias is None else s + bias.float()
    M, E = c.shape
    if n_group and n_group > 1:
        gs = c.view(M, n_group, E // n_group).topk(2, dim=-1)[0].sum(dim=-1)
        gidx = torch.topk(gs, k=topk_group, dim=-1)[1]
        gmask = torch.zeros_like(gs, dtype=torch.bool).scatter_(1, gidx, True)
        emask = gmask.unsqueeze(-1).expand(M, n_group, E // n_group).reshape(M, E)
        c = c.masked_fill(~emask, float("-inf"))
    ids = torch.topk(c, K, dim=-1)[1]
    w = s.gather(1, ids)
    w = w / (w.sum(dim=-1, keepdim=True) + 1e-20) * scale
    return w, ids.to(torch.int32)


# -------------------------------------------------------------------- align
def align(ids: torch.Tensor, E: int):
    """moe_pre_sorted index outputs: stable sort of the flat ids by expert."""
    flat = ids.reshape(-1).long()
    sorted_src = torch.sort(flat, stable=True)[1]
    moe_index = torch.empty_like(sorted_src)
    moe_index[sorted_src] = torch.arange(flat.numel())
    expert_m = torch.bincount(flat, minlength=E)
    lod = torch.zeros(E + 1, dtype=torch.long)
    lod[1:] = torch.cumsum(expert_m, 0)
    return moe_index.int(), sorted_src.int(), expert_m.int(), lod.int()


# -------------------------------------------------------------------- quant
def quant_i8_rows(x: torch.Tensor):
    """quant2d: per-row absmax int8; returns (q int8, max f32 [R,1])."""
    xf = x.float()
    mx = xf.abs().amax(dim=-1, keepdim=True)
    inv = torch.where(mx > 0, 127.0 / mx, torch.zeros_like(mx))
    q = torch.round(xf * inv).clamp_(-127, 127).to(torch.int8)
    return q, mx


def quantize_weight_per_channel(w: torch.Tensor):
    """Per-output-channel symmetric int8 of a float weight [..., n, k]:
    returns (int8 weight, scale [..., n, 1]); the layer stores max = 127*scale
    after process_weights_after_loading (compressed_tensors_moe.py:116-120)."""
    mx = w.float().abs().amax(dim=-1, keepdim=True).clamp_min(1e-12)
    q = torch.round(w.float() * (127.0 / mx)).clamp_(-127, 127).to(torch.int8)
    return q, mx / 127.0


def _int8_mm(a: torch.Tensor, b_t: torch.Tensor) -> torch.Tensor:
    """a [m,k] int8 times b_t [n,k]^T -> int32 [m,n], exact."""
    if a.shape[0] == 0:
        return torch.zeros(0, b_t.shape[0], dtype=torch.int32)
    return torch._int_mm(a.contiguous(), b_t.t())


def _dequant(acc: torch.Tensor, a_max: torch.Tensor, w_max: torch.Tensor, dtype) -> torch.Tensor:
    """acc * (a_max/127) * (w_max/127) -> activation dtype."""
    return ((acc.float() * (a_max.float() / 127.0)) * (w_max.float().reshape(1, -1) / 127.0)).to(dtype)


def silu_and_mul(y: torch.Tensor) -> torch.Tensor:
    d = y.shape[-1] // 2
    return (F.silu(y[..., :d].float()) * y[..., d:].float()).to(y.dtype)


# ------------------------------------------------------------ layer: W8A8
def route(logits, K, scoring="softmax", renormalize=True, n_group=1, topk_group=1, routed_scale=1.0, bias=None):
    if scoring == "softmax":
        return softmax_topk(logits, K, renormalize)
    return sigmoid_group_topk_norm(logits, bias, K, n_group, topk_group, routed_scale)


def w8a8_dense(x, w13, w13_max, w2, w2_max):
    """Dense W8A8 MLP (the shared expert): scaled_int8_quant -> matmul with
    x_pc_max / w_pc_max (quantization/kernels/scale_mm.py:63-90), twice."""
    xq, xmax = quant_i8_rows(x)
    y = _dequant(_int8_mm(xq, w13), xmax, w13_max, x.dtype)
    a = silu_and_mul(y)
    aq, amax = quant_i8_rows(a)
    return _dequant(_int8_mm(aq, w2), amax, w2_max, x.dtype)


def w8a8_moe(x, logits, w13, w13_max, w2, w2_max, K, scoring="softmax", renormalize=True, n_group=1, topk_group=1,
             routed_scale=1.0, bias=None, shared=None, out_scale=1.0, topk=None):
    """The reference's torch expert loop with the W8A8 stage arithmetic.
    x [M,H] bf16; w13 [E,2I,H] int8 with max [E,2I,1]; w2 [E,H,I] int8 with max [E,H,1]."""
    M, H = x.shape
    E = w13.shape[0]
    w, ids = topk if topk is not None else route(logits, K, scoring, renormalize, n_group, topk_group, routed_scale,
                                                 bias)
    out = torch.zeros(M * K, H, dtype=x.dtype)
    repeat_x = x.repeat_interleave(K, dim=0)
    flat = ids.reshape(-1)
    for e in range(E):
        sel = flat == e
        if sel.sum():
            cur = repeat_x[sel]
            xq, xmax = quant_i8_rows(cur)
            y = _dequant(_int8_mm(xq, w13[e]), xmax, w13_max[e], x.dtype)
            a = silu_and_mul(y)
            aq, amax = quant_i8_rows(a)
            out[sel] = _dequant(_int8_mm(aq, w2[e]), amax, w2_max[e], x.dtype)
    res = (out.view(M, K, H).float() * w.float().unsqueeze(2)).sum(dim=1).to(x.dtype)
    if out_scale != 1.0:
        res = res * out_scale
    if shared is not None:
        res = res + w8a8_dense(x, *shared)
    return res


# ------------------------------------------------------------ layer: bf16
def bf16_moe(x, logits, w13, w2, K, renormalize=True, ep_rank=0):
    """KunlunOps.fused_moe_ep restated line for line in meaning
    (ops/_kunlun_ops.py:655-696): weights cast to the activation dtype, product
    and sum over K in that dtype. The weights are the local experts of rank ep_rank
    (global ids ep_rank * num_local_experts + i, :677-678); logits run over all experts."""
    M, H = x.shape
    E = w13.shape[0]
    w, ids = softmax_topk(logits, K, False)
    if renormalize:
        w = w / w.sum(1, keepdim=True)
    w = w.to(x.dtype)
    out = torch.zeros(M * K, H, dtype=x.dtype)
    repeat_x = x.repeat_interleave(K, dim=0)
    flat = ids.reshape(-1)
    for e in range(E):
        sel = flat == ep_rank * E + e
        if sel.sum():
            cur = repeat_x[sel]
            out[sel] = silu_and_mul(cur @ w13[e].T) @ w2[e].T
    return (out.view(M, K, H) * w.unsqueeze(2)).sum(dim=1).to(x.dtype)


def swigluoai_and_mul(x: torch.Tensor, alpha: float = 1.702, limit: float = 7.0) -> torch.Tensor:
    """torch.ops._C.swigluoai_and_mul as the reference defines it (ops/_custom_ops.py:728-742)."""
    gate, up = x[..., ::2], x[..., 1::2]
    gate = gate.clamp(min=None, max=limit)
    up = up.clamp(min=-limit, max=limit)
    glu = gate * torch.sigmoid(gate * alpha)
    return (up + 1) * glu


def bf16_moe_bias(x, logits, w13, w2, w13_bias, w2_bias, K, alpha: float = 1.702, limit: float = 7.0):
    """The expert-bias (gpt-oss) branch of KunlunOps.fused_moe restated line for line in meaning
    (ops/_kunlun_ops.py:433-468): routing weights cast to the activation dtype, per-expert
    `x @ w1.T + b1`, swigluoai, `@ w2.T + b2`, weighted sum over K in that dtype."""
    M, H = x.shape
    E = w13.shape[0]
    w, ids = softmax_topk(logits, K, True)
    w = w.to(x.dtype)
    out = torch.zeros(M * K, H, dtype=x.dtype)
    repeat_x = x.repeat_interleave(K, dim=0)
    flat = ids.reshape(-1)
    for e in range(E):
        sel = flat == e
        if sel.sum():
            g1 = repeat_x[sel] @ w13[e].T
            if w13_bias is not None:
                g1 = g1 + w13_bias[e]
            up_gate = swigluoai_and_mul(g1, alpha, limit)
            g2 = up_gate @ w2[e].T
            if w2_bias is not None:
                g2 = g2 + w2_bias[e]
            out[sel] = g2
    return (out.view(M, K, H) * w.unsqueeze(2)).sum(dim=1).to(x.dtype)


# -------------------------------------------------------------- fp8 (c5)
FP8_MAX = 448.0


def quant_fp8_group128(x: torch.Tensor):
    """Per-row, per-128-column e4m3fn: scale = absmax/448, q = e4m3fn(x/scale)."""
    R, Cc = x.shape
    xf = x.float().view(R, Cc // 128, 128)
    s = xf.abs().amax(dim=-1, keepdim=True) / FP8_MAX
    y = torch.where(s > 0, xf / s, torch.zeros_like(xf)).clamp_(-FP8_MAX, FP8_MAX)
    return y.to(torch.float8_e4m3fn).view(R, Cc), s.squeeze(-1)


def quantize_weight_fp8_block128(w: torch.Tensor):
    """[..., n, k] float -> e4m3fn with one f32 scale per 128x128 block [..., n/128, k/128]."""
    *lead, n, k = w.shape
    wf = w.float().reshape(*lead, n // 128, 128, k // 128, 128)
    s = wf.abs().amax(dim=(-3, -1), keepdim=True).clamp_min(1e-12) / FP8_MAX
    q = (wf / s).clamp_(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn).reshape(*lead, n, k)
    return q, s.reshape(*lead, n // 128, k // 128)


def fp8_block_gemm(aq, a_scale, wq, w_scale, dtype=torch.bfloat16):
    """sum over 128-wide K blocks of (q_a . q_w^T) * s_a[r,kb] * s_w[n/128,kb], f32."""
    R, k = aq.shape
    n = wq.shape[0]
    af = aq.float().view(R, k // 128, 128)
    wf = wq.float().view(n, k // 128, 128)
    part = torch.einsum("rbk,nbk->rnb", af, wf)
    ws = w_scale.float().repeat_interleave(128, dim=0)[:n]  # [n, k/128]
    return (part * a_scale.float().unsqueeze(1) * ws.unsqueeze(0)).sum(-1).to(dtype)
