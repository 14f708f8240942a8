"""MoE gate projection (reference: vllm_kunlun/ops/fused_moe/router/gate_linear.py:10-116).

The reference picks between a DeepSeek-V3 special kernel, a bf16 x bf16 -> fp32 library
GEMM and F.linear; here there is one kernel (kmoe_router_gemm_bf16: bf16 operands, f32
accumulation and output, split K for small batches), and a caller that wants the
logits never to leave the layer passes `gate.weight` to
`apply_monolithic(..., router_logits=None, router_weight=gate.weight)` instead.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import layer as _layer  # noqa: F401  (keeps the package import order of the reference)
from ... import _custom_ops  # noqa: F401  (registers torch.ops._C.router_gemm_bf16_fp32)


class GateLinear(torch.nn.Module):
    """`forward(x) -> (logits, None)` like ReplicatedLinear; weight [num_experts, hidden] bf16 (or float16, the model's dtype)."""

    def __init__(self, input_size: int, output_size: int, bias: bool = False,
                 out_dtype: Optional[torch.dtype] = None, params_dtype: Optional[torch.dtype] = None,
                 force_fp32_compute: bool = False, prefix: str = "", device=None):
        super().__init__()
        if bias:
            raise NotImplementedError("GateLinear: bias is not supported (the reference's MoE gates have none)")
        if params_dtype not in (None, torch.bfloat16, torch.float16):
            raise NotImplementedError(f"GateLinear: weights must be bfloat16 or float16, got {params_dtype}")
        self.weight = torch.nn.Parameter(torch.zeros(output_size, input_size, dtype=params_dtype or torch.bfloat16,
                                                     device=device), requires_grad=False)
        self.out_dtype = out_dtype
        self.prefix = prefix
        self.e_score_correction_bias = None

    def set_out_dtype(self, out_dtype: torch.dtype) -> None:
        if self.out_dtype is not None:
            raise ValueError("out_dtype has already been set")
        self.out_dtype = out_dtype

    def forward(self, x: torch.Tensor):
        if x.dtype != self.weight.dtype:
            x = x.to(self.weight.dtype)
        logits = torch.ops._C.router_gemm_bf16_fp32(x, self.weight)
        if self.out_dtype is not None and self.out_dtype != torch.float32:
            logits = logits.to(self.out_dtype)
        return logits, None
