"""FusedMoE layer holder and the unquantized (bf16) monolithic method.

vLLM is not a dependency of this package, so `FusedMoE` / `SharedFusedMoE` here
are small stand-ins that carry exactly the attributes the reference's methods
read from vLLM's layer (reference: vllm_kunlun/ops/fused_moe/layer.py:50-80,
compressed_tensors_moe.py:135-138, models/deepseek_v2.py:241-261) and call the
quant method the way vLLM's FusedMoE.forward_impl does for a monolithic method:
`quant_method.apply_monolithic(layer, x, router_logits)`.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch


@dataclass
class FusedMoEConfig:
    """The fields of vLLM's FusedMoEConfig that the methods read through `self.moe`."""
    experts_per_token: int
    num_experts: int = 0
    hidden_dim: int = 0
    use_ep: bool = False
    ep_rank: int = 0


class KunlunUnquantizedFusedMoEMethod:
    """bf16 weights, monolithic entry (reference: ops/fused_moe/layer.py:16-81)."""

    def __init__(self, moe: FusedMoEConfig):
        self.moe = moe

    @property
    def is_monolithic(self) -> bool:
        return True

    def create_weights(self, layer, num_experts, hidden_size, intermediate_size_per_partition,
                       params_dtype=torch.bfloat16, device=None, **_):
        E, H, I = num_experts, hidden_size, intermediate_size_per_partition
        layer.w13_weight = torch.nn.Parameter(torch.zeros(E, 2 * I, H, dtype=params_dtype, device=device),
                                              requires_grad=False)
        layer.w2_weight = torch.nn.Parameter(torch.zeros(E, H, I, dtype=params_dtype, device=device),
                                             requires_grad=False)

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        """Nothing to repack (the reference skips upstream's Triton kernel set-up here)."""

    def apply_monolithic(self, layer, x: torch.Tensor, router_logits: torch.Tensor):
        from .._kunlun_ops import KunlunOps as ops
        common = dict(renormalize=layer.renormalize, inplace=True, use_grouped_topk=layer.use_grouped_topk,
                      num_expert_group=layer.num_expert_group, topk_group=layer.topk_group)
        if self.moe.use_ep:
            return ops.fused_moe_ep(x, layer.w13_weight, layer.w2_weight, router_logits, self.moe.ep_rank,
                                    self.moe.experts_per_token, **common)
        return ops.fused_moe(x, layer.w13_weight, layer.w2_weight, router_logits, self.moe.ep_rank,
                             self.moe.experts_per_token, scoring_func=layer.scoring_func,
                             e_score_correction_bias=layer.e_score_correction_bias,
                             w1_bias=getattr(layer, "w13_bias", None), w2_bias=getattr(layer, "w2_bias", None),
                             **common)


class FusedMoE(torch.nn.Module):
    """Attribute-compatible stand-in for vLLM's FusedMoE."""

    def __init__(self, num_experts: int, top_k: int, hidden_size: int, intermediate_size: int,
                 params_dtype: torch.dtype = torch.bfloat16, renormalize: bool = True,
                 use_grouped_topk: bool = False, num_expert_group: Optional[int] = None,
                 topk_group: Optional[int] = None, scoring_func: str = "softmax",
                 routed_scaling_factor: float = 1.0, e_score_correction_bias: Optional[torch.Tensor] = None,
                 quant_method=None, device=None):
        super().__init__()
        self.global_num_experts = num_experts
        self.top_k = top_k
        self.hidden_size = hidden_size
        self.intermediate_size_per_partition = intermediate_size
        self.renormalize = renormalize
        self.use_grouped_topk = use_grouped_topk
        self.num_expert_group = num_expert_group
        self.topk_group = topk_group
        self.scoring_func = scoring_func
        self.routed_scaling_factor = routed_scaling_factor
        self.e_score_correction_bias = e_score_correction_bias
        self.moe_config = FusedMoEConfig(experts_per_token=top_k, num_experts=num_experts, hidden_dim=hidden_size)
        self.quant_method = quant_method if quant_method is not None else KunlunUnquantizedFusedMoEMethod(
            self.moe_config)
        if getattr(self.quant_method, "moe", None) is None:
            self.quant_method.moe = self.moe_config
        self.quant_method.create_weights(self, num_experts, hidden_size, intermediate_size, params_dtype,
                                         device=device)

    def forward(self, hidden_states: torch.Tensor, router_logits: torch.Tensor):
        if not self.quant_method.is_monolithic:
            raise RuntimeError("only monolithic MoE methods are served by this build")
        return self.quant_method.apply_monolithic(self, hidden_states, router_logits)


class SharedFusedMoE(FusedMoE):
    """FusedMoE plus a dense shared expert evaluated on the same input; returns
    (shared_output, routed_output) like upstream's SharedFusedMoE
    (reference use: models/deepseek_v2.py:241-284)."""

    def __init__(self, shared_experts: Optional[torch.nn.Module], **kwargs):
        super().__init__(**kwargs)
        self.shared_experts = shared_experts

    def forward(self, hidden_states: torch.Tensor, router_logits: torch.Tensor):
        routed = super().forward(hidden_states, router_logits)
        shared = self.shared_experts(hidden_states) if self.shared_experts is not None else None
        return shared, routed
