"""Quantized fused-MoE methods: the plugin-level entry of the path.

Mirrors the interface of the reference's
vllm_kunlun/quantization/compressed_tensors/compressed_tensors_moe.py
(KunlunCompressedTensorsMoEMethod.get_moe_method :43-108,
KunlunCompressedTensorsW8A8Int8MoEMethod :111-291): `is_monolithic`,
`process_weights_after_loading(layer)` and
`apply_monolithic(layer, x, router_logits, ...)`, same argument meaning, same
exceptions. Where the reference launches nine closed kernels and allocates every
intermediate per call, `apply_monolithic` here makes ONE call into libkmoe
(kmoe_moe_forward) on a cached workspace.
"""
from __future__ import annotations

from typing import Optional, Union

import torch

from ... import _lib as L
from ..._plan import MoEPlan, make_moe_plan, tile_pair_, tile_w4_scales_
from ...ops import _custom_ops  # noqa: F401  (torch.ops._C.* used by the staged path)

WNA16_SUPPORTED_BITS = (4, 8)
W8A8Plan = MoEPlan  # the plan type returned by make_plan


def _get(o, k, d=None):
    return o.get(k, d) if isinstance(o, dict) else getattr(o, k, d)


def _strategy(o) -> str:
    return str(_get(o, "strategy")).split(".")[-1].lower()


def _scheme_is_dynamic_token_w8a8(weight_quant, input_quant) -> bool:
    """compressed-tensors "int-quantized" W8A8: 8-bit symmetric channel/tensor
    weights, 8-bit symmetric dynamic per-token activations."""
    if weight_quant is None or input_quant is None:
        return False
    return (_get(weight_quant, "num_bits") == 8 and _get(input_quant, "num_bits") == 8
            and str(_get(weight_quant, "type", "int")).split(".")[-1].lower() == "int"
            and _strategy(weight_quant) in ("channel", "tensor") and _strategy(input_quant) == "token"
            and bool(_get(weight_quant, "symmetric", True)) and bool(_get(input_quant, "symmetric", True))
            and bool(_get(input_quant, "dynamic", False)) and not bool(_get(weight_quant, "dynamic", False)))


def _scheme_is_fp8_block(weight_quant, input_quant) -> bool:
    """8-bit float weights in 128x128 blocks, dynamic per-token-group(128) float activations."""
    if weight_quant is None or input_quant is None:
        return False
    return (_get(weight_quant, "num_bits") == 8 and _get(input_quant, "num_bits") == 8
            and str(_get(weight_quant, "type", "int")).split(".")[-1].lower() == "float"
            and _strategy(weight_quant) == "block" and list(_get(weight_quant, "block_structure", [])) == [128, 128]
            and _strategy(input_quant) == "group" and _get(input_quant, "group_size") == 128
            and bool(_get(input_quant, "dynamic", False)))


def _scheme_is_wna16(weight_quant, input_quant) -> bool:
    if weight_quant is None or input_quant is not None:
        return False
    return _strategy(weight_quant) in ("channel", "group")


class KunlunCompressedTensorsMoEMethod:
    """Scheme dispatcher (reference: compressed_tensors_moe.py:42-108)."""

    @staticmethod
    def get_moe_method(quant_config, layer: torch.nn.Module, layer_name: str):
        if hasattr(quant_config, "_add_fused_moe_to_target_scheme_map"):
            quant_config._add_fused_moe_to_target_scheme_map()
        unfused = [layer_name + p for p in (".0.gate_proj", ".0.up_proj", ".0.down_proj")]
        schemes = [quant_config.get_scheme_dict(layer, name) for name in unfused]
        scheme = schemes.pop()
        if not all(s == scheme for s in schemes):
            raise ValueError("All MoE projections need to have same quantization scheme but found multiple")
        if scheme is None:  # ignored layer
            from ...ops.fused_moe.layer import KunlunUnquantizedFusedMoEMethod
            return KunlunUnquantizedFusedMoEMethod(layer.moe_config)
        weight_quant = scheme.get("weights")
        input_quant = scheme.get("input_activations")
        if _scheme_is_wna16(weight_quant, input_quant):
            fmt = scheme.get("format")
            if _get(weight_quant, "num_bits") != 4 or fmt not in (None, "pack-quantized"):
                raise ValueError(f"For Fused MoE layers, only format pack-quantized and 4 bits is supported but got "
                                 f"format: {fmt} and bits: {_get(weight_quant, 'num_bits')}")
            return KunlunCompressedTensorsWNA16MoEMethod(weight_quant, input_quant, layer.moe_config)
        if _scheme_is_dynamic_token_w8a8(weight_quant, input_quant):
            return KunlunCompressedTensorsW8A8Int8MoEMethod(weight_quant, input_quant, layer.moe_config)
        if _scheme_is_fp8_block(weight_quant, input_quant):
            return KunlunCompressedTensorsW8A8Fp8MoEMethod(weight_quant, input_quant, layer.moe_config)
        raise RuntimeError(f"Unsupported FusedMoe scheme: {weight_quant}, {input_quant}")


class _MonolithicQuantMoE:
    """What the int8 and fp8 methods share: routing-argument resolution and the plan."""

    FORMAT = None

    def __init__(self, weight_quant=None, input_quant=None, moe=None):
        self.weight_quant = weight_quant
        self.input_quant = input_quant
        self.moe = moe

    @property
    def is_monolithic(self) -> bool:
        return True

    # True: a shared expert that cannot ride in the routed launches may run on the library's second stream beside
    # them (KMOE_FLAG_SIDE_STREAM). Off by default: every launch then goes to the current stream, as the
    # reference's does.
    side_stream = False

    # routing parameters: kwargs win; a kwarg left at its default falls back to the layer
    @staticmethod
    def _routing(layer, topk_group, num_expert_group, scoring_func, routed_scaling_factor, bias):
        if scoring_func == "softmax" and getattr(layer, "scoring_func", "softmax") != "softmax":
            scoring_func = layer.scoring_func
        if topk_group is None:
            topk_group = getattr(layer, "topk_group", None)
        if num_expert_group is None:
            num_expert_group = getattr(layer, "num_expert_group", None)
        if bias is None:
            bias = getattr(layer, "e_score_correction_bias", None)
        if routed_scaling_factor == 1.0:
            routed_scaling_factor = float(getattr(layer, "routed_scaling_factor", 1.0) or 1.0)
        if scoring_func not in ("softmax", "sigmoid"):
            raise ValueError(f"Unsupported scoring_func: {scoring_func}")
        return topk_group, num_expert_group, scoring_func, routed_scaling_factor, bias

    def apply_monolithic(
        self,
        layer: torch.nn.Module,
        x: torch.Tensor,
        router_logits: torch.Tensor,
        topk_group: Optional[int] = None,
        num_expert_group: Optional[int] = None,
        global_num_experts: int = -1,
        scoring_func: str = "softmax",
        routed_scaling_factor: float = 1.0,
        e_score_correction_bias: Optional[torch.Tensor] = None,
        shared_expert=None,
        out_scale: float = 1.0,
        router_weight: Optional[torch.Tensor] = None,
        shared_scale: float = 1.0,
    ) -> Union[torch.Tensor, tuple]:
        """x [M,H] bf16 or float16, router_logits [M,E] -> [M,H] in x's dtype
        (reference: :122-291).
        `shared_expert` (w13, w13_max, w2, w2_max of a dense MLP in the layer's format), `out_scale` and
        `shared_scale` fold the caller's epilogue (models/deepseek_v2.py:286-296) into the call:
        `routed * out_scale + shared * shared_scale`, i.e. (routed_scaling_factor, 1) for bfloat16 and
        (1, 1 / routed_scaling_factor) for float16, which the reference scales that way round against overflow;
        with `router_logits=None` and `router_weight` (the [E,H] weight of the gate in x's dtype,
        models/deepseek_v2.py:178-184) the gate projection of :275 runs inside the call too."""
        if x.dtype not in (torch.bfloat16, torch.float16):
            raise NotImplementedError(f"apply_monolithic: activations must be bfloat16 or float16, got {x.dtype}")
        x = x.contiguous()
        logits = None if router_logits is None else router_logits.float().contiguous()
        out = torch.empty((x.shape[0], layer.w2_weight.shape[1]), dtype=x.dtype, device=x.device)
        plan = self.make_plan(layer, x, logits, out, topk_group, num_expert_group, scoring_func,
                              routed_scaling_factor, e_score_correction_bias, shared_expert, out_scale,
                              router_weight=router_weight, shared_scale=shared_scale)
        plan()
        self.last_layout, self.last_workspace = plan.layout, plan.workspace  # lets tests read the intermediates
        return out

    def make_plan(self, layer, x, logits, out, topk_group=None, num_expert_group=None, scoring_func="softmax",
                  routed_scaling_factor=1.0, e_score_correction_bias=None, shared_expert=None, out_scale=1.0,
                  stage_events=None, router_weight=None, shared_scale=1.0) -> MoEPlan:
        """Argument block for repeated calls on fixed buffers (x bf16 [M,H], logits f32
        [M,E], out bf16 [M,H], all contiguous): what a serving loop or a HIP-graph
        capture replays without touching Python-side allocation."""
        topk_group, num_expert_group, scoring_func, routed_scaling_factor, bias = self._routing(
            layer, topk_group, num_expert_group, scoring_func, routed_scaling_factor, e_score_correction_bias)
        # Under expert parallelism the layer holds the experts of one rank while the logits (or the router weight)
        # run over all of them: the rank's share, as KunlunOps.fused_moe_ep computes it for the unquantized layer
        # (ops/_kunlun_ops.py:677-689). The reference's own quantized path takes the local experts for all (:135).
        E = layer.w13_weight.shape[0]
        routed = logits.shape[-1] if logits is not None else router_weight.shape[0]
        first = int(getattr(self.moe, "ep_rank", 0) or 0) * E if routed > E else 0
        return make_moe_plan(self.FORMAT, x, logits, out, self.moe.experts_per_token, layer.w13_weight,
                             layer.w2_weight, layer.w13_weight_scale, layer.w2_weight_scale, scoring_func,
                             True,  # the reference always routes with the *_norm kernels
                             num_expert_group, topk_group, routed_scaling_factor, bias, shared_expert, out_scale,
                             stage_events, router_weight=router_weight, shared_scale=shared_scale, first_expert=first,
                             side_stream=bool(self.side_stream))


class KunlunCompressedTensorsW8A8Int8MoEMethod(_MonolithicQuantMoE):
    """Dynamic-per-token W8A8 int8 MoE (reference: compressed_tensors_moe.py:111-291)."""

    FORMAT = L.KMOE_FMT_INT8

    def create_weights(self, layer: torch.nn.Module, num_experts: int, hidden_size: int,
                       intermediate_size_per_partition: int, params_dtype: torch.dtype = torch.bfloat16,
                       device=None, **_) -> None:
        """Parameters as upstream's W8A8 int8 MoE method creates them: int8 weights
        and one f32 SCALE per output channel (shapes per compressed_tensors_moe.py:135-137,212,258)."""
        E, H, I = num_experts, hidden_size, intermediate_size_per_partition
        mk = lambda *s, dt: torch.nn.Parameter(torch.zeros(*s, dtype=dt, device=device), requires_grad=False)  # noqa
        layer.w13_weight = mk(E, 2 * I, H, dt=torch.int8)
        layer.w2_weight = mk(E, H, I, dt=torch.int8)
        layer.w13_weight_scale = mk(E, 2 * I, 1, dt=torch.float32)
        layer.w2_weight_scale = mk(E, H, 1, dt=torch.float32)

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        """scale -> absmax: the kernels dequantise with max/127 (reference: :116-120).
        On the GPU the int8 weights are also re-arranged in place into MFMA-ready blocks
        (same values, same results; see kmoe_tile_weights_i8) when both shapes allow it."""
        with torch.no_grad():
            layer.w13_weight_scale.mul_(127.0)
            layer.w2_weight_scale.mul_(127.0)
            if getattr(self, "tile_weights", True):
                if getattr(self, "pad_intermediate", True):
                    self._pad_intermediate_(layer)
                tile_pair_(layer.w13_weight, layer.w2_weight)

    # the blocks of tiled weights hold 64 bytes of K: the down projection's K is the intermediate size
    PAD_MULTIPLE = 64

    @classmethod
    def _pad_intermediate_(cls, layer: torch.nn.Module) -> bool:
        """An intermediate size that is not a multiple of 64 (96 = 768 / 8 on a tensor-parallel
        shard, 160, ...) would keep both weights row-major, on the slow kernels. Pads it with
        zero channels instead: gate rows [0, I), up rows [I', I' + I) of w13, columns [0, I) of
        w2, zero weights and zero absmax elsewhere. A padded channel's accumulator is 0, its
        SiLU-mul output 0, its code 0 and its weight in w2 0: the layer's output keeps every bit.
        The parameters are replaced (shapes [E, 2I', H], [E, 2I', 1], [E, H, I']); the original
        size stays in `layer.intermediate_size_unpadded`. Returns whether it padded."""
        w13, w2, s13 = layer.w13_weight.data, layer.w2_weight.data, layer.w13_weight_scale.data
        E, two_i, H = w13.shape
        I = two_i // 2
        Ip = -(-I // cls.PAD_MULTIPLE) * cls.PAD_MULTIPLE
        if Ip == I or not w13.is_cuda or w13.dtype != torch.int8 or H % 64 or tuple(w2.shape) != (E, H, I):
            return False
        w13p = torch.zeros((E, 2 * Ip, H), dtype=w13.dtype, device=w13.device)
        w13p[:, :I].copy_(w13[:, :I])
        w13p[:, Ip:Ip + I].copy_(w13[:, I:])
        s13p = torch.zeros((E, 2 * Ip) + tuple(s13.shape[2:]), dtype=s13.dtype, device=s13.device)
        s13p[:, :I].copy_(s13[:, :I])
        s13p[:, Ip:Ip + I].copy_(s13[:, I:])
        w2p = torch.zeros((E, H, Ip), dtype=w2.dtype, device=w2.device)
        w2p[:, :, :I].copy_(w2)
        layer.w13_weight = torch.nn.Parameter(w13p, requires_grad=False)
        layer.w13_weight_scale = torch.nn.Parameter(s13p, requires_grad=False)
        layer.w2_weight = torch.nn.Parameter(w2p, requires_grad=False)
        layer.intermediate_size_unpadded = I
        return True

    def apply_staged(self, layer, x, router_logits, topk_group=None, num_expert_group=None, global_num_experts=-1,
                     scoring_func="softmax", routed_scaling_factor=1.0, e_score_correction_bias=None):
        """The same layer through the operator-level surface, one torch.ops._C.* call
        per stage in the reference's order (compressed_tensors_moe.py:139-291).
        Bit-identical to apply_monolithic; kept for callers that drive the ops themselves."""
        topk_group, num_expert_group, scoring_func, routed_scaling_factor, bias = self._routing(
            layer, topk_group, num_expert_group, scoring_func, routed_scaling_factor, e_score_correction_bias)
        ops = torch.ops._C
        E, two_i, H = layer.w13_weight.shape
        M, K, dev = x.shape[0], self.moe.experts_per_token, x.device
        normed_score = torch.empty(M, K, dtype=torch.float32, device=dev)
        topk_ids = torch.empty(M, K, dtype=torch.int32, device=dev)
        block_statistic = torch.zeros(12, E, dtype=torch.int32, device=dev)
        logits = router_logits.float()
        if scoring_func == "softmax":
            ops.moe_softmax_topk_norm(logits, normed_score, topk_ids, None, True)
        else:
            ops.moe_sigmoid_group_topk_norm(logits, topk_ids, normed_score, block_statistic, bias,
                                            routed_scaling_factor, num_expert_group, topk_group)
        if M * K > 768:
            moe_expand = torch.empty(M * K, H, dtype=x.dtype, device=dev)
            expert_m = torch.zeros(E, dtype=torch.int32, device=dev)
            lod = torch.zeros(E + 1, dtype=torch.int32, device=dev)
            sorted_tokens_idx = torch.zeros(M * K, dtype=torch.int32, device=dev)
            ops.gen_block_statistic(topk_ids, block_statistic)
            ops.moe_pre_sorted(x, topk_ids, block_statistic, moe_expand, sorted_tokens_idx, expert_m, lod)
        else:
            sorted_tokens_idx, lod, moe_expand = torch.ops.xspeedgate_ops.moe_pre_small(topk_ids, E, False, True, x)
        y = torch.empty(M, K, two_i, dtype=x.dtype, device=dev)
        x_q = torch.empty(M * K, H, dtype=torch.int8, device=dev)
        x_scale = torch.empty(M * K, 1, dtype=torch.float32, device=dev)
        ops.quant2d(moe_expand, x_q, x_scale, True)
        ops.moe_fc(x_q, layer.w13_weight, lod, sorted_tokens_idx, K, y, None, x_scale, layer.w13_weight_scale,
                   topk_ids)
        out1 = torch.empty(M, K, two_i // 2, dtype=x.dtype, device=dev)
        ops.silu_and_mul(out1, y)
        out1 = out1.reshape(-1, two_i // 2)
        x_q = torch.empty(out1.shape, dtype=torch.int8, device=dev)
        x_scale = torch.empty(out1.shape[0], 1, dtype=torch.float32, device=dev)
        ops.quant2d(out1, x_q, x_scale, True)
        out = torch.empty(M, K, H, dtype=x.dtype, device=dev)
        ops.moe_fc(x_q, layer.w2_weight, lod, sorted_tokens_idx, K, out, None, x_scale, layer.w2_weight_scale,
                   topk_ids)
        dequant_scale = torch.ones(M, K, dtype=torch.float32, device=dev)
        output = torch.empty(M, H, dtype=x.dtype, device=dev)
        ops.moe_post(out, sorted_tokens_idx.view(M, K), normed_score, dequant_scale, output)
        return output


class KunlunCompressedTensorsW8A8Fp8MoEMethod(_MonolithicQuantMoE):
    """fp8-e4m3fn weights with 128x128 block scales, dynamic per-token-group(128) fp8
    activations (DeepSeek-V3 recipe). No counterpart in the reference, whose platform
    rejects fp8 (platforms/kunlun.py:350-364); same monolithic interface as the int8 method."""

    FORMAT = L.KMOE_FMT_FP8_BLOCK

    def create_weights(self, layer: torch.nn.Module, num_experts: int, hidden_size: int,
                       intermediate_size_per_partition: int, params_dtype: torch.dtype = torch.bfloat16,
                       device=None, **_) -> None:
        E, H, I = num_experts, hidden_size, intermediate_size_per_partition
        if H % 128 or I % 128:
            raise ValueError("fp8 block-scaled MoE needs hidden and intermediate sizes that are multiples of 128")
        mk = lambda *s, dt: torch.nn.Parameter(torch.zeros(*s, dtype=dt, device=device), requires_grad=False)  # noqa
        layer.w13_weight = mk(E, 2 * I, H, dt=torch.float8_e4m3fn)
        layer.w2_weight = mk(E, H, I, dt=torch.float8_e4m3fn)
        layer.w13_weight_scale = mk(E, 2 * I // 128, H // 128, dt=torch.float32)
        layer.w2_weight_scale = mk(E, H // 128, I // 128, dt=torch.float32)

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        """Block scales are used as they are (dequant = code * scale). On the GPU the e4m3 codes
        are re-arranged in place into the same MFMA-ready 1 KB blocks as int8 weights."""
        if getattr(self, "tile_weights", True):
            with torch.no_grad():
                tile_pair_(layer.w13_weight, layer.w2_weight)


class KunlunCompressedTensorsWNA16MoEMethod:
    """4-bit weight-only MoE (reference: compressed_tensors_moe.py:294-360). The reference
    unpacks the whole packed weight tensors to fp16 inside EVERY apply() (:320-327) and then
    calls the unquantized fused_moe. Here, in process_weights_after_loading:
      * the packed tensors are tiled in place and kept for kmoe_grouped_gemm_w4a16, which unpacks in
        registers (a weight-streaming kernel for decode-sized batches, a kernel on 64- to 128-row tiles beyond;
        needs hidden and intermediate sizes that are multiples of 128 and a group size that is a multiple
        of 32);
      * or the weights are unpacked ONCE (kmoe_dequant_w4) to tiled 16-bit tensors for the unquantized path.
    `native` chooses: "auto" (default) keeps the packed tensors alone where the kernels take the shapes (a
    quarter of the 16-bit bytes; measured on the Qwen3-30B-A3B shape against the 16-bit copy: 0.10 against
    0.22 ms at 128 tokens, 0.21 against 0.26 ms at 1024, 0.50 against 0.45 ms at 4096, 0.86 against 0.76 ms at
    8192) and the 16-bit copy alone elsewhere; "both" keeps both (1.25x the 16-bit bytes) and takes the faster
    one per batch; "only" is "auto" that refuses shapes the packed kernels do not take; False never uses the
    packed kernels.
    The 16-bit type is the one of the scales: float16 scales (a model loaded with --dtype float16, the
    reference's recipes) give half((code - 8) * scale), exactly what dequant_int4_native computes, and the
    layer then takes float16 activations; any other scale dtype is taken as bfloat16.
    Packed layout as in dequant_int4_native (quantization/kernels/quant_ops.py:71-86): uint8,
    two codes per byte, low nibble first, code - 8; scales per contiguous group of `group_size`
    along k, or one per row."""

    # native="both": rows per expert up to which the packed weights are used (above: the unpacked copy). Measured
    # cross-over on the Qwen3-30B-A3B shape: between 2048 tokens (128 rows per expert: 0.33 against 0.33 ms) and
    # 4096 (256 rows: 0.50 against 0.45 ms).
    NATIVE_MAX_ROWS_PER_EXPERT = 160

    def __init__(self, weight_quant=None, input_quant=None, moe=None, native="auto"):
        self.weight_quant = weight_quant
        self.input_quant = input_quant
        self.moe = moe
        gs = _get(weight_quant, "group_size") if weight_quant is not None else None
        self.group_size = int(gs) if (gs and _strategy(weight_quant) == "group") else None  # None: one scale per row
        if native not in ("auto", "both", "only", False):
            raise ValueError("native must be 'auto', 'both', 'only' or False")
        self.native = native

    @property
    def is_monolithic(self) -> bool:
        return True

    def create_weights(self, layer: torch.nn.Module, num_experts: int, hidden_size: int,
                       intermediate_size_per_partition: int, params_dtype: torch.dtype = torch.bfloat16,
                       device=None, **_) -> None:
        E, H, I = num_experts, hidden_size, intermediate_size_per_partition
        if H % 16 or I % 16:
            raise ValueError("4-bit MoE weights need hidden and intermediate sizes that are multiples of 16")
        g13 = H // self.group_size if self.group_size else 1
        g2 = I // self.group_size if self.group_size else 1
        mk = lambda *s, dt: torch.nn.Parameter(torch.zeros(*s, dtype=dt, device=device), requires_grad=False)  # noqa
        layer.w13_weight_packed = mk(E, 2 * I, H // 2, dt=torch.uint8)
        layer.w2_weight_packed = mk(E, H, I // 2, dt=torch.uint8)
        sdt = torch.float16 if params_dtype == torch.float16 else torch.bfloat16
        layer.w13_weight_scale = mk(E, 2 * I, g13, dt=sdt)
        layer.w2_weight_scale = mk(E, H, g2, dt=sdt)

    def _native_possible(self, layer) -> bool:
        E, n13, half_h = layer.w13_weight_packed.shape
        H, I = 2 * half_h, n13 // 2
        gs13, gs2 = self.group_size or H, self.group_size or I
        return (layer.w13_weight_packed.is_cuda and H % 128 == 0 and I % 128 == 0 and gs13 == gs2
                and gs13 % 32 == 0 and H % gs13 == 0 and I % gs13 == 0)

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        with torch.no_grad():
            native = self.native and self._native_possible(layer)
            if self.native == "only" and not native:
                raise ValueError("native='only' needs CUDA tensors, H and I multiples of 128 and one group size "
                                 "(a multiple of 32) for both weight tensors")
            keep_bf16 = self.native == "both" or not native
            for name in ("w13", "w2"):
                packed = getattr(layer, f"{name}_weight_packed").data.contiguous()
                scale = getattr(layer, f"{name}_weight_scale").data
                dt16 = torch.float16 if layer.w13_weight_scale.dtype == torch.float16 else torch.bfloat16
                scale = scale.to(dt16).contiguous()
                E, n, half_k = packed.shape
                k = 2 * half_k
                gs = self.group_size or k
                if k % gs or scale.shape[-1] != k // gs:
                    raise ValueError(f"{name}: scales {tuple(scale.shape)} do not fit k={k}, group_size={gs}")
                L.require_device(packed, scale)
                if keep_bf16:
                    w = torch.empty((E, n, k), dtype=dt16, device=packed.device)
                    L.check(L.lib.kmoe_dequant_w4(L.ptr(packed), L.ptr(scale), E * n, k, gs, L.ptr(w),
                                                  L.act_dtype(w), L.stream()))
                    setattr(layer, f"{name}_weight", torch.nn.Parameter(w, requires_grad=False))
                if native:
                    getattr(layer, f"{name}_weight_packed").data = packed
                    getattr(layer, f"{name}_weight_scale").data = scale
                else:
                    delattr(layer, f"{name}_weight_packed")
            if native:
                if not tile_pair_(layer.w13_weight_packed, layer.w2_weight_packed):
                    raise RuntimeError("4-bit weights: tiling the packed tensors failed")
                # the scales too: per 16 channels [groups][16], so that what a block needs is one piece of memory
                if not (tile_w4_scales_(layer.w13_weight_scale) and tile_w4_scales_(layer.w2_weight_scale)):
                    raise RuntimeError("4-bit weights: re-arranging the group scales failed")
            layer.w4_native = bool(native)
            if keep_bf16 and getattr(self, "tile_weights", True):
                tile_pair_(layer.w13_weight, layer.w2_weight)

    def _routing_kwargs(self, layer):
        return dict(scoring_func=getattr(layer, "scoring_func", "softmax"),
                    num_expert_group=getattr(layer, "num_expert_group", None),
                    topk_group=getattr(layer, "topk_group", None),
                    e_score_correction_bias=getattr(layer, "e_score_correction_bias", None))

    def apply_monolithic(self, layer, x: torch.Tensor, router_logits: torch.Tensor, **kwargs):
        """The layer-driven call: top_k from the method's `moe`, routing attributes from the layer."""
        return self._run(layer, x, router_logits, self.moe.experts_per_token, **self._routing_kwargs(layer))

    def apply(self, layer: torch.nn.Module, x: torch.Tensor, router_logits: torch.Tensor, top_k: int, renormalize: bool,
              use_grouped_topk: bool = False, topk_group: Optional[int] = None, num_expert_group: Optional[int] = None,
              global_num_experts: int = -1, expert_map: Optional[torch.Tensor] = None, custom_routing_function=None,
              scoring_func: str = "softmax", routed_scaling_factor: float = 1.0,
              e_score_correction_bias: Optional[torch.Tensor] = None, apply_router_weight_on_input: bool = False,
              activation: str = "silu", enable_eplb: bool = False, expert_load_view: Optional[torch.Tensor] = None,
              logical_to_physical_map: Optional[torch.Tensor] = None,
              logical_replica_count: Optional[torch.Tensor] = None):
        """The reference's entry point, argument for argument (compressed_tensors_moe.py:296-360). As there, what
        reaches the computation is top_k, scoring_func, the group arguments and the correction bias: `renormalize`,
        `use_grouped_topk` and `routed_scaling_factor` stop at KunlunOps.fused_moe, which always normalises and
        uses scale 1.0 (_kunlun_ops.py:385-431). Arguments the reference accepts and ignores but which would change
        the result if honoured are refused rather than ignored."""
        if expert_map is not None or custom_routing_function is not None or apply_router_weight_on_input or enable_eplb:
            raise NotImplementedError("4-bit MoE: expert_map, custom_routing_function, apply_router_weight_on_input "
                                      "and EPLB are not on this path")
        if activation != "silu":
            raise NotImplementedError(f"4-bit MoE: activation {activation!r} (silu only)")
        if getattr(self.moe, "use_ep", False):
            # the expert-parallel branch (:329-342) ends in KunlunOps.fused_moe_ep: softmax routing over the experts of
            # router_logits' width, `renormalize` honoured, the layer's weights being those of rank ep_rank
            return self._run(layer, x, router_logits, top_k, renormalize=bool(renormalize),
                             ep_rank=int(getattr(self.moe, "ep_rank", 0)))
        return self._run(layer, x, router_logits, top_k, scoring_func=scoring_func, num_expert_group=num_expert_group,
                         topk_group=topk_group, e_score_correction_bias=e_score_correction_bias)

    def _run(self, layer, x, router_logits, top_k, scoring_func="softmax", num_expert_group=None, topk_group=None,
             e_score_correction_bias=None, renormalize=True, ep_rank=None):
        """Activations in the dtype of the scales (bf16, or float16). On the packed weights:
        kmoe_grouped_gemm_w4a16 inside kmoe_moe_forward. On the unpacked copy: KunlunOps.fused_moe, as
        the reference's apply() ends (:343-360). Routing as in KunlunOps.fused_moe (always
        normalised, sigmoid scale 1.0)."""
        E = layer.w13_weight_scale.shape[0] if getattr(layer, "w4_native", False) else layer.w13_weight.shape[0]
        rows_per_expert = -(-x.shape[0] * top_k // E)
        has_bias = getattr(layer, "w13_bias", None) is not None or getattr(layer, "w2_bias", None) is not None
        use_native = getattr(layer, "w4_native", False) and not has_bias and (
            self.native != "both" or rows_per_expert <= self.NATIVE_MAX_ROWS_PER_EXPERT)
        if use_native:
            if x.dtype != layer.w13_weight_scale.dtype:
                raise ValueError(f"4-bit MoE: activations ({x.dtype}) must have the dtype of the scales "
                                 f"({layer.w13_weight_scale.dtype})")
            xc = x.contiguous()
            out = torch.empty_like(xc)
            gs = self.group_size or 2 * layer.w13_weight_packed.shape[-1]
            plan = make_moe_plan(L.KMOE_FMT_W4A16, xc, router_logits.to(torch.float).contiguous(), out, top_k,
                                 layer.w13_weight_packed, layer.w2_weight_packed, layer.w13_weight_scale,
                                 layer.w2_weight_scale, scoring_func, renormalize, num_expert_group, topk_group, 1.0,
                                 e_score_correction_bias, group_size=gs, first_expert=(ep_rank or 0) * E)
            plan()
            return out
        if not hasattr(layer, "w13_weight"):
            raise NotImplementedError("4-bit MoE: expert biases need the unpacked copy (native='both' or False)")
        from ...ops._kunlun_ops import KunlunOps as ops
        if ep_rank is not None:  # the expert-parallel entry: its own routing (softmax, `renormalize` honoured)
            return ops.fused_moe_ep(x, layer.w13_weight, layer.w2_weight, router_logits, ep_rank, top_k,
                                    renormalize=renormalize, inplace=True)
        return ops.fused_moe(x, layer.w13_weight, layer.w2_weight, router_logits, 0, top_k,
                             renormalize=getattr(layer, "renormalize", True), inplace=True,
                             use_grouped_topk=getattr(layer, "use_grouped_topk", False),
                             num_expert_group=num_expert_group, topk_group=topk_group, scoring_func=scoring_func,
                             e_score_correction_bias=e_score_correction_bias,
                             w1_bias=getattr(layer, "w13_bias", None), w2_bias=getattr(layer, "w2_bias", None))
