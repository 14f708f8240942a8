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
    """bf16 (or float16) weights in the activations' dtype, monolithic entry (reference: ops/fused_moe/layer.py:16-81)."""

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
        """The reference skips upstream's Triton kernel set-up here; on the GPU this build
        re-arranges the bf16 weights in place into MFMA-ready blocks (same values)."""
        from ..._plan import tile_pair_
        if getattr(self, "tile_weights", True):
            with torch.no_grad():
                tile_pair_(layer.w13_weight, layer.w2_weight)

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

    # ---- checkpoint -> parameters (reference use: models/deepseek_v2.py:1285-1384) ----
    @classmethod
    def make_expert_params_mapping(cls, ckpt_gate_proj_name: str, ckpt_down_proj_name: str,
                                   ckpt_up_proj_name: str, num_experts: int,
                                   num_redundant_experts: int = 0) -> list[tuple[str, str, int, str]]:
        """(param_name, weight_name, expert_id, shard_id) for every expert projection, as the
        model's load_weights expects (models/deepseek_v2.py:1296-1302): a checkpoint tensor
        whose name contains `weight_name` ("experts.7.up_proj.") belongs to the stacked
        parameter named by replacing that piece with `param_name` ("experts.w13_"), at
        expert 7, shard w3. Redundant experts (expert-parallel load balancing) are not
        served on one GPU."""
        if num_redundant_experts:
            raise NotImplementedError("redundant experts belong to expert parallelism, which this build does not span")
        out = []
        for e in range(num_experts):
            for shard_id, proj in (("w1", ckpt_gate_proj_name), ("w2", ckpt_down_proj_name), ("w3", ckpt_up_proj_name)):
                param = "experts.w13_" if shard_id in ("w1", "w3") else "experts.w2_"
                out.append((param, f"experts.{e}.{proj}.", e, shard_id))
        return out

    def weight_loader(self, param: torch.nn.Parameter, loaded_weight: torch.Tensor, weight_name: str,
                      shard_id: str, expert_id: int, return_success: bool = False):
        """Copies one projection (or its scales) of one expert into the stacked parameter:
        w1 -> rows [0, n/2) of w13 (gate), w3 -> rows [n/2, n) (up), w2 -> all of w2. Row
        counts follow the parameter, so weights [2I,H], per-channel scales [2I,1] and block
        scales [2I/128, H/128] all load through here. Must run BEFORE
        process_weights_after_loading (which re-tiles the codes in place)."""
        if shard_id not in ("w1", "w2", "w3"):
            raise ValueError(f"shard_id must be w1, w2 or w3, got {shard_id}")
        from ..._plan import is_tiled
        if is_tiled(param):
            raise RuntimeError("weight_loader: this parameter was already re-tiled by process_weights_after_loading")
        if not 0 <= expert_id < param.shape[0]:
            return False if return_success else None
        dst = param.data[expert_id]
        if shard_id != "w2":
            half = dst.shape[0] // 2
            dst = dst[:half] if shard_id == "w1" else dst[half:]
        src = loaded_weight
        if src.dim() == dst.dim() - 1:  # per-channel scales stored as [n]
            src = src.unsqueeze(-1)
        if tuple(src.shape) != tuple(dst.shape):
            raise ValueError(f"{weight_name}: checkpoint tensor {tuple(loaded_weight.shape)} does not fit "
                             f"{tuple(dst.shape)} (expert {expert_id}, shard {shard_id})")
        if src.dtype != dst.dtype and src.element_size() == 1 and dst.element_size() == 1:
            src = src.view(dst.dtype)  # e4m3 codes stored as uint8
        dst.copy_(src)
        return True if return_success else None

    def load_weights(self, weights, ckpt_gate_proj_name: str = "gate_proj", ckpt_down_proj_name: str = "down_proj",
                     ckpt_up_proj_name: str = "up_proj") -> set:
        """Loads every tensor of `weights` (an iterable of (name, tensor), e.g. from safetensors)
        that names an expert projection of this layer: "...experts.<e>.<proj>.weight",
        ".weight_scale". Returns the names consumed; other names are left to the caller."""
        mapping = self.make_expert_params_mapping(ckpt_gate_proj_name, ckpt_down_proj_name, ckpt_up_proj_name,
                                                  self.global_num_experts)
        by_piece = {weight_name: (param_name, e, shard) for param_name, weight_name, e, shard in mapping}
        params = dict(self.named_parameters())
        loaded = set()
        for name, tensor in weights:
            i = name.find("experts.")
            if i < 0:
                continue
            parts = name[i:].split(".")  # experts, <e>, <proj>, <suffix...>
            if len(parts) < 4 or not parts[1].isdigit():
                continue
            piece = ".".join(parts[:3]) + "."
            if piece not in by_piece:
                continue
            param_name, e, shard = by_piece[piece]
            target = param_name.split(".", 1)[1] + ".".join(parts[3:])  # "w13_" + "weight_scale"
            if target not in params:
                continue
            self.weight_loader(params[target], tensor, name, shard_id=shard, expert_id=e)
            loaded.add(name)
        return loaded


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
