"""Seeded synthetic MoE layers of the benchmark shapes.

Weights ~ N(0, 0.02) quantised per output channel to int8 (scale = absmax/127),
activations ~ N(0, 1) bf16, router logits ~ N(0, 1) f32, correction bias
~ N(0, 0.01). Everything is generated on the target device from one seeded
generator, expert by expert, so the 11 GB DeepSeek-V3-shape layer never needs a
float copy of itself; tests copy back to the host whatever their checker needs.
"""
from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Optional

import torch

from .ops.fused_moe.layer import FusedMoE
from .quantization.compressed_tensors.compressed_tensors_moe import KunlunCompressedTensorsW8A8Int8MoEMethod


@dataclass(frozen=True)
class MoEShape:
    name: str
    M: int            # tokens
    H: int            # hidden
    E: int            # routed experts
    K: int            # experts per token
    I: int            # moe intermediate
    scoring: str = "softmax"
    n_group: int = 1
    topk_group: int = 1
    routed_scale: float = 1.0
    I_shared: int = 0  # intermediate of the dense shared expert (0: none)
    hot_experts: int = 0   # add +hot_bias to the logits of this many fixed experts
    hot_bias: float = 0.0
    quant: str = "int8"    # "none" (bf16 weights), "int8", "fp8", "w4" (4-bit weights, bf16 activations)
    group_size: int = 128  # "w4": values per weight scale

    @property
    def P(self) -> int:
        return self.M * self.K


# The benchmark configurations (tokens are the decode / prefill batch of each).
SHAPES = {
    "tiny-bf16": MoEShape("tiny-bf16", 32, 512, 8, 2, 256, quant="none"),
    "qwen3-decode": MoEShape("qwen3-decode", 64, 2048, 128, 8, 768),
    "qwen3-prefill": MoEShape("qwen3-prefill", 8192, 2048, 128, 8, 768),
    "qwen3-prefill-skew": MoEShape("qwen3-prefill-skew", 8192, 2048, 128, 8, 768, hot_experts=8, hot_bias=2.0),
    "dsv3-decode": MoEShape("dsv3-decode", 128, 7168, 256, 8, 2048, "sigmoid", 8, 4, 2.5, 2048),
    "dsv3-prefill": MoEShape("dsv3-prefill", 4096, 7168, 256, 8, 2048, "sigmoid", 8, 4, 2.5, 2048),
    "kimi-decode": MoEShape("kimi-decode", 128, 7168, 384, 8, 2048, "sigmoid", 1, 1, 2.5, 2048),
    "kimi-prefill": MoEShape("kimi-prefill", 4096, 7168, 384, 8, 2048, "sigmoid", 1, 1, 2.5, 2048),
}
# the same layers with fp8-e4m3 block-scaled weights (128x128 blocks) and per-token-group activations
for _n in ("dsv3-decode", "dsv3-prefill", "kimi-decode", "kimi-prefill"):
    _f = _n.replace("-", "-fp8-")
    SHAPES[_f] = replace(SHAPES[_n], name=_f, quant="fp8")


# the Qwen3 layers unquantized (bf16 weights): what KunlunOps.fused_moe serves
for _n in ("qwen3-decode", "qwen3-prefill"):
    _f = _n.replace("-", "-bf16-")
    SHAPES[_f] = replace(SHAPES[_n], name=_f, quant="none")


# ... and with 4-bit weights (group scales of 128 values) on the packed-weight paths
SHAPES["qwen3-w4a16-decode"] = replace(SHAPES["qwen3-decode"], name="qwen3-w4a16-decode", quant="w4")
SHAPES["qwen3-w4a16-prefill"] = replace(SHAPES["qwen3-prefill"], name="qwen3-w4a16-prefill", quant="w4")
# the Kimi-K2 dimensions with 4-bit routed experts in groups of 32 (the shared expert of such a checkpoint stays a
# 16-bit dense layer of its own, outside this layer)
for _n in ("kimi-decode", "kimi-prefill"):
    _f = _n.replace("-", "-w4a16-")
    SHAPES[_f] = replace(SHAPES[_n], name=_f, quant="w4", group_size=32, I_shared=0)


def make_layer(shape: MoEShape, device="cuda", seed: int = 0, dtype: torch.dtype = torch.bfloat16) -> "SynthLayer":
    """The synthetic layer of a shape in the format the shape names. dtype: bfloat16, or float16 (int8: the
    and fp8: the activations; unquantized: activations and weights; 4-bit: activations and group scales)."""
    if dtype == torch.bfloat16:
        return {"int8": make_w8a8_layer, "fp8": make_fp8_layer, "none": make_bf16_layer,
                "w4": make_w4_layer}[shape.quant](shape, device, seed)
    if dtype != torch.float16:
        raise NotImplementedError(f"synthetic {shape.quant} layer with {dtype} activations")
    if shape.quant in ("int8", "fp8"):
        sl = (make_w8a8_layer if shape.quant == "int8" else make_fp8_layer)(shape, device, seed)
        return SynthLayer(sl.shape, sl.layer, sl.x.half(), sl.logits, sl.bias, sl.shared)
    return {"none": make_bf16_layer, "w4": make_w4_layer}[shape.quant](shape, device, seed, dtype)


def scaled(shape: MoEShape, **kw) -> MoEShape:
    """A copy of a shape with some fields replaced (reduced sizes for CPU-checkable tests)."""
    return replace(shape, **kw)


def _quant_rows_int8(w: torch.Tensor):
    mx = w.abs().amax(dim=-1, keepdim=True).clamp_min(1e-12)
    q = torch.round(w * (127.0 / mx)).clamp_(-127, 127).to(torch.int8)
    return q, mx / 127.0


@dataclass
class SynthLayer:
    shape: MoEShape
    layer: FusedMoE
    x: torch.Tensor                 # [M,H] bf16
    logits: torch.Tensor            # [M,E] f32
    bias: Optional[torch.Tensor]    # [E] f32 (sigmoid routing)
    shared: Optional[tuple]         # (ws13 i8 [2Is,H], ws13_max f32 [2Is], ws2 i8 [H,Is], ws2_max f32 [H])

    def host_weights(self):
        """(w13, w13_aux, w2, w2_aux, shared) as host tensors in the reference's row-major
        layout (int8 weights are un-tiled), for a CPU checker."""
        from ._plan import rowmajor_int8_weights, rowmajor_w4_scales
        lay = self.layer

        def rm(t):
            return rowmajor_int8_weights(t).detach().cpu()

        def aux(name):  # (the group scales of packed 4-bit weights are re-arranged at load time as well)
            if not hasattr(lay, name):
                return None
            t = getattr(lay, name)
            return (rowmajor_w4_scales(t) if t.dtype in (torch.bfloat16, torch.float16) else t).detach().cpu()

        shared = None
        if self.shared is not None:
            shared = (rm(self.shared[0]), self.shared[1].detach().cpu(), rm(self.shared[2]),
                      self.shared[3].detach().cpu())
        packed = not hasattr(lay, "w13_weight")  # 4-bit layer that kept only its packed weights
        return (rm(lay.w13_weight_packed if packed else lay.w13_weight), aux("w13_weight_scale"),
                rm(lay.w2_weight_packed if packed else lay.w2_weight), aux("w2_weight_scale"), shared)

    def apply_kwargs(self) -> dict:
        s = self.shape
        kw = dict(scoring_func=s.scoring)
        if s.scoring == "sigmoid":
            kw.update(num_expert_group=s.n_group, topk_group=s.topk_group, routed_scaling_factor=s.routed_scale,
                      e_score_correction_bias=self.bias)
        if self.shared is not None:
            kw["shared_expert"] = self.shared
        return kw


def rebatch(sl: SynthLayer, shape: MoEShape, seed: int = 0) -> SynthLayer:
    """Another batch for the same weights: a SynthLayer that shares `sl`'s layer, correction bias and
    shared expert and carries fresh activations and router logits of `shape` (its tokens, its hot
    experts), drawn from a generator seeded with (seed, tokens)."""
    a, b = sl.shape, shape
    same = ("H", "E", "K", "I", "scoring", "n_group", "topk_group", "routed_scale", "I_shared", "quant", "group_size")
    if any(getattr(a, f) != getattr(b, f) for f in same):
        raise ValueError("rebatch: the new shape must keep the layer's dimensions, routing and format")
    dev = sl.x.device
    g = torch.Generator(device=dev)
    g.manual_seed(seed * 1000003 + shape.M)
    x, logits = _activations(shape, g, dev)
    return SynthLayer(shape, sl.layer, x.to(sl.x.dtype), logits, sl.bias, sl.shared)


def _quant_block_fp8(w: torch.Tensor):
    """[n,k] float -> e4m3fn codes + one f32 scale per 128x128 block (absmax/448)."""
    n, k = w.shape
    wb = w.reshape(n // 128, 128, k // 128, 128)
    s = wb.abs().amax(dim=(1, 3), keepdim=True).clamp_min(1e-12) / 448.0
    q = (wb / s).clamp_(-448.0, 448.0).to(torch.float8_e4m3fn).reshape(n, k)
    return q, s.reshape(n // 128, k // 128)


def _routing_inputs(s: MoEShape, g, dev):
    bias = None
    if s.scoring == "sigmoid":
        bias = torch.randn(s.E, generator=g, device=dev, dtype=torch.float32) * 0.01
    return bias


def _activations(s: MoEShape, g, dev):
    x = torch.randn(s.M, s.H, generator=g, device=dev).to(torch.bfloat16)
    logits = torch.randn(s.M, s.E, generator=g, device=dev, dtype=torch.float32)
    if s.hot_experts:
        hot = torch.arange(s.hot_experts, device=dev) * (s.E // s.hot_experts)
        logits[:, hot] += s.hot_bias
    return x, logits


def make_fp8_layer(shape: MoEShape, device="cuda", seed: int = 0) -> SynthLayer:
    """FusedMoE with the fp8 block-scaled method and random weights quantised per 128x128 block."""
    from .quantization.compressed_tensors.compressed_tensors_moe import KunlunCompressedTensorsW8A8Fp8MoEMethod
    dev = torch.device(device)
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    s = shape
    method = KunlunCompressedTensorsW8A8Fp8MoEMethod()
    bias = _routing_inputs(s, g, dev)
    layer = FusedMoE(num_experts=s.E, top_k=s.K, hidden_size=s.H, intermediate_size=s.I, renormalize=True,
                     use_grouped_topk=s.n_group > 1, num_expert_group=s.n_group, topk_group=s.topk_group,
                     scoring_func=s.scoring, e_score_correction_bias=bias, quant_method=method, device=dev)
    for e in range(s.E):
        q, sc = _quant_block_fp8(torch.randn(2 * s.I, s.H, generator=g, device=dev) * 0.02)
        layer.w13_weight.data[e].copy_(q)
        layer.w13_weight_scale.data[e].copy_(sc)
        q, sc = _quant_block_fp8(torch.randn(s.H, s.I, generator=g, device=dev) * 0.02)
        layer.w2_weight.data[e].copy_(q)
        layer.w2_weight_scale.data[e].copy_(sc)
    method.process_weights_after_loading(layer)
    shared = None
    if s.I_shared:
        q13, s13 = _quant_block_fp8(torch.randn(2 * s.I_shared, s.H, generator=g, device=dev) * 0.02)
        q2, s2 = _quant_block_fp8(torch.randn(s.H, s.I_shared, generator=g, device=dev) * 0.02)
        shared = (q13, s13.contiguous(), q2, s2.contiguous())
        from ._plan import is_tiled, tile_pair_
        if is_tiled(layer.w13_weight):
            tile_pair_(q13, q2)
    x, logits = _activations(s, g, dev)
    return SynthLayer(s, layer, x, logits, bias, shared)


def make_bf16_layer(shape: MoEShape, device="cuda", seed: int = 0, dtype: torch.dtype = torch.bfloat16) -> SynthLayer:
    """FusedMoE with the unquantized method and bf16 (or float16) weights ~ N(0, 0.02)."""
    dev = torch.device(device)
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    s = shape
    bias = _routing_inputs(s, g, dev)
    layer = FusedMoE(num_experts=s.E, top_k=s.K, hidden_size=s.H, intermediate_size=s.I, renormalize=True,
                     use_grouped_topk=s.n_group > 1, num_expert_group=s.n_group, topk_group=s.topk_group,
                     scoring_func=s.scoring, e_score_correction_bias=bias, device=dev, params_dtype=dtype)
    for e in range(s.E):
        layer.w13_weight.data[e].copy_(torch.randn(2 * s.I, s.H, generator=g, device=dev) * 0.02)
        layer.w2_weight.data[e].copy_(torch.randn(s.H, s.I, generator=g, device=dev) * 0.02)
    layer.quant_method.process_weights_after_loading(layer)
    x, logits = _activations(s, g, dev)
    return SynthLayer(s, layer, x.to(dtype), logits, bias, None)


def make_w4_layer(shape: MoEShape, device="cuda", seed: int = 0, dtype: torch.dtype = torch.bfloat16) -> SynthLayer:
    """FusedMoE with the 4-bit method (packed weights alone, native="only"): weights ~ N(0, 0.02)
    quantised per group of `group_size` values to codes 0..15 (value = (code - 8) * scale)."""
    from types import SimpleNamespace
    from .quantization.compressed_tensors.compressed_tensors_moe import KunlunCompressedTensorsWNA16MoEMethod
    dev = torch.device(device)
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    s = shape
    bias = _routing_inputs(s, g, dev)
    wq = SimpleNamespace(num_bits=4, type="int", symmetric=True, dynamic=False, strategy="group",
                         group_size=s.group_size)
    method = KunlunCompressedTensorsWNA16MoEMethod(wq, None, SimpleNamespace(experts_per_token=s.K), native="only")
    layer = FusedMoE(num_experts=s.E, top_k=s.K, hidden_size=s.H, intermediate_size=s.I, renormalize=True,
                     use_grouped_topk=s.n_group > 1, num_expert_group=s.n_group, topk_group=s.topk_group,
                     scoring_func=s.scoring, e_score_correction_bias=bias, quant_method=method, device=dev,
                     params_dtype=dtype)

    def quantise(w):  # [n, k] float -> packed uint8 [n, k/2], 16-bit scales [n, k/gs]
        n, k = w.shape
        grp = w.view(n, k // s.group_size, s.group_size)
        scale = (grp.abs().amax(-1) / 7.0).clamp_min(1e-6).to(dtype)
        codes = (torch.round(grp / scale.float().unsqueeze(-1)).clamp(-8, 7) + 8).to(torch.uint8).view(n, k)
        return codes[:, 0::2] | (codes[:, 1::2] << 4), scale

    for e in range(s.E):
        p13, s13 = quantise(torch.randn(2 * s.I, s.H, generator=g, device=dev) * 0.02)
        p2, s2 = quantise(torch.randn(s.H, s.I, generator=g, device=dev) * 0.02)
        layer.w13_weight_packed.data[e].copy_(p13)
        layer.w13_weight_scale.data[e].copy_(s13)
        layer.w2_weight_packed.data[e].copy_(p2)
        layer.w2_weight_scale.data[e].copy_(s2)
    method.process_weights_after_loading(layer)
    x, logits = _activations(s, g, dev)
    return SynthLayer(s, layer, x.to(dtype), logits, bias, None)


def make_w8a8_layer(shape: MoEShape, device="cuda", seed: int = 0) -> SynthLayer:
    """Builds a FusedMoE with the W8A8 method, fills it with quantised random
    weights and runs process_weights_after_loading (scales become maxes)."""
    dev = torch.device(device)
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    s = shape
    method = KunlunCompressedTensorsW8A8Int8MoEMethod()
    bias = None
    if s.scoring == "sigmoid":
        bias = torch.randn(s.E, generator=g, device=dev, dtype=torch.float32) * 0.01
    layer = FusedMoE(num_experts=s.E, top_k=s.K, hidden_size=s.H, intermediate_size=s.I,
                     renormalize=True, use_grouped_topk=s.n_group > 1, num_expert_group=s.n_group,
                     topk_group=s.topk_group, scoring_func=s.scoring, e_score_correction_bias=bias,
                     quant_method=method, device=dev)
    for e in range(s.E):
        q, sc = _quant_rows_int8(torch.randn(2 * s.I, s.H, generator=g, device=dev) * 0.02)
        layer.w13_weight.data[e].copy_(q)
        layer.w13_weight_scale.data[e].copy_(sc)
        q, sc = _quant_rows_int8(torch.randn(s.H, s.I, generator=g, device=dev) * 0.02)
        layer.w2_weight.data[e].copy_(q)
        layer.w2_weight_scale.data[e].copy_(sc)
    method.process_weights_after_loading(layer)
    shared = None
    if s.I_shared:
        q13, s13 = _quant_rows_int8(torch.randn(2 * s.I_shared, s.H, generator=g, device=dev) * 0.02)
        q2, s2 = _quant_rows_int8(torch.randn(s.H, s.I_shared, generator=g, device=dev) * 0.02)
        shared = (q13, (s13 * 127.0).reshape(-1).contiguous(), q2, (s2 * 127.0).reshape(-1).contiguous())
        from ._plan import is_tiled, tile_pair_
        if is_tiled(layer.w13_weight):  # the shared expert goes through the same load-time step
            tile_pair_(q13, q2)
    x = torch.randn(s.M, s.H, generator=g, device=dev).to(torch.bfloat16)
    logits = torch.randn(s.M, s.E, generator=g, device=dev, dtype=torch.float32)
    if s.hot_experts:
        hot = torch.arange(s.hot_experts, device=dev) * (s.E // s.hot_experts)
        logits[:, hot] += s.hot_bias
    return SynthLayer(s, layer, x, logits, bias, shared)
