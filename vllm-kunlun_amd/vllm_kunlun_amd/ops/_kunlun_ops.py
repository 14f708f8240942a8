"""`KunlunOps`: the static façade the reference's MoE methods call, MoE part only.

Mirrors `KunlunOps.fused_moe` and `KunlunOps.fused_moe_ep` of
vllm_kunlun/ops/_kunlun_ops.py (:377-637 and :639-696): same argument lists, same
return value ([M,H] in the activation dtype). Both run the unquantized (bf16)
layer as one call into libkmoe (kmoe_moe_forward, KMOE_FMT_BF16); the reference's
device pipeline and its torch expert loop compute the same function.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import _lib as L
from .._plan import make_moe_plan


class KunlunOps:
    @staticmethod
    def fused_moe(
        hidden_states: torch.Tensor,
        w1: torch.Tensor,
        w2: torch.Tensor,
        router_logits: torch.Tensor,
        ep_rank: int,
        moe_top_k: int,
        renormalize: bool,
        inplace: bool = False,
        use_grouped_topk: bool = False,
        num_expert_group: Optional[int] = None,
        topk_group: Optional[int] = None,
        w1_bias: Optional[torch.Tensor] = None,
        w2_bias: Optional[torch.Tensor] = None,
        scoring_func: str = "softmax",
        e_score_correction_bias: Optional[torch.Tensor] = None,
    ) -> torch.Tensor:
        """Unquantized (bf16 or float16) fused MoE (reference: ops/_kunlun_ops.py:377-637). As there, routing is
        chosen by `scoring_func` alone and always normalises (`renormalize`,
        `use_grouped_topk` and `inplace` are accepted and ignored, :385-389 vs :413-431);
        the sigmoid path uses scale 1.0 (:428)."""
        L.act_dtype(hidden_states, "fused_moe")  # bfloat16 or float16; the weights must match
        x = hidden_states.contiguous()
        logits = router_logits.to(torch.float).contiguous()
        out = torch.empty_like(x)
        extra = {}
        if w1_bias is not None or w2_bias is not None:
            # the gpt-oss branch (:433-468): per-expert biases, gate/up interleaved, swigluoai_and_mul
            extra = dict(w13_bias=None if w1_bias is None else w1_bias.to(torch.bfloat16).contiguous(),
                         w2_bias=None if w2_bias is None else w2_bias.to(torch.bfloat16).contiguous(),
                         activation="swigluoai")
        plan = make_moe_plan(L.KMOE_FMT_BF16, x, logits, out, moe_top_k, w1, w2, None, None, scoring_func, True,
                             num_expert_group, topk_group, 1.0, e_score_correction_bias, **extra)
        plan()
        return out

    @staticmethod
    def fused_moe_ep(
        hidden_states: torch.Tensor,
        w13_weight: torch.Tensor,
        w2_weight: torch.Tensor,
        router_logits: torch.Tensor,
        ep_rank: int,
        top_k: int,
        renormalize: bool,
        inplace: bool = False,
        use_grouped_topk: bool = False,
        num_expert_group: Optional[int] = None,
        topk_group: Optional[int] = None,
        w1_bias: Optional[torch.Tensor] = None,
        w2_bias: Optional[torch.Tensor] = None,
    ) -> torch.Tensor:
        """The expert-parallel entry (reference: ops/_kunlun_ops.py:639-696): softmax routing over the experts of
        router_logits' width, `renormalize` honoured (:670-671); the weights are the num_local_experts experts from
        ep_rank * num_local_experts on (:677-678), and the result is what the pairs routed to them contribute -
        the caller's all-reduce over the ranks makes the layer's output, as in the reference."""
        L.act_dtype(hidden_states, "fused_moe_ep")
        x = hidden_states.contiguous()
        logits = router_logits.to(torch.float).contiguous()
        out = torch.empty_like(x)
        plan = make_moe_plan(L.KMOE_FMT_BF16, x, logits, out, top_k, w13_weight, w2_weight, None, None, "softmax",
                             bool(renormalize), first_expert=int(ep_rank) * w13_weight.shape[0])
        plan()
        return out
