"""Dense W8A8 linear layer (the shared expert's gate_up and down projections, and any other
int8 Linear of a W8A8 checkpoint).

Mirror of `KunlunScaledMMLinearKernel` (reference: quantization/kernels/scale_mm.py:30-90), which
vLLM's `CompressedTensorsW8A8Int8` scheme instantiates per Linear. The reference derives from
vLLM's `CutlassInt8ScaledMMLinearKernel`; vLLM is not a dependency here, so this class carries the
few pieces of that base it relies on (the parameter names and what the base's
`process_weights_after_loading` leaves behind: the weight as the [k, n] transpose view of its
[n, k] storage, a per-channel weight scale, no input scale for dynamic quantisation).

Path taken by `apply_weights`: per-token absmax int8 quantisation (`_C::scaled_int8_quant`) and the
one-expert case of the grouped int8 GEMM on the weights re-arranged at load time into the MFMA
tiles (`kmoe_grouped_gemm_i8`), the same kernels the fused MoE layer runs its shared expert on.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from ... import _lib as L
from ..._plan import is_tiled, tile_int8_weights_


@dataclass
class Int8ScaledMMLinearLayerConfig:
    """The fields of vLLM's config of the same name that the kernel selection reads."""
    is_channelwise: bool = True
    is_static_input_scheme: bool = False
    input_symmetric: bool = True


class KunlunScaledMMLinearKernel:
    def __init__(self, c: Optional[Int8ScaledMMLinearLayerConfig] = None, w_q_param_name: str = "weight",
                 w_s_param_name: str = "weight_scale", i_s_param_name: str = "input_scale",
                 i_zp_param_name: str = "input_zero_point", azp_adj_param_name: str = "azp_adj"):
        self.config = c or Int8ScaledMMLinearLayerConfig()
        self.layer_param_names = (w_q_param_name, w_s_param_name, i_s_param_name, i_zp_param_name,
                                  azp_adj_param_name)
        self._lod = {}  # (device, rows) -> the {0, rows} row range of the single expert, made once

    @classmethod
    def is_supported(cls, compute_capability: Optional[int] = None) -> tuple[bool, Optional[str]]:
        """Reference: scale_mm.py:32-37 (there: any out-of-tree platform). Here: a HIP device."""
        if not torch.cuda.is_available():
            return False, "requires a HIP device."
        return True, None

    @classmethod
    def can_implement(cls, c: Int8ScaledMMLinearLayerConfig) -> tuple[bool, Optional[str]]:
        """Reference: scale_mm.py:39-41 accepts every config and fails later; this class says up
        front which schemes its kernels cover."""
        if c.is_static_input_scheme:
            return False, "static (per-tensor) input scales are not implemented; dynamic per-token only."
        if not c.input_symmetric:
            return False, "asymmetric activations (azp) are not implemented."
        return True, None

    def _get_layer_params(self, layer):
        return tuple(getattr(layer, name, None) for name in self.layer_param_names)

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        """Base-class part: the weight parameter becomes the [k, n] transpose view, the weight
        scale one f32 per output channel. Reference part (scale_mm.py:43-50): scale -> absmax
        (x 127), in place. Added here: the [n, k] storage is re-arranged into the MFMA tiles once
        (when n % 16 == 0 and k % 64 == 0) and kept on the layer for `apply_weights`."""
        w_q_name, w_s_name, i_s_name, i_zp_name, azp_adj_name = self.layer_param_names
        weight = getattr(layer, w_q_name)
        w_nk = weight.data
        if w_nk.dtype != torch.int8 or w_nk.dim() != 2:
            raise ValueError(f"{w_q_name}: expected int8 [n, k], got {w_nk.dtype} {tuple(w_nk.shape)}")
        w_nk = w_nk.contiguous()
        n, k = w_nk.shape
        w_s = getattr(layer, w_s_name)
        scale = w_s.data.to(torch.float32).reshape(-1)
        if scale.numel() == 1:  # per-tensor scale of an unfused layer -> one per channel
            scale = scale.expand(n)
        if scale.numel() != n:
            raise ValueError(f"{w_s_name}: {scale.numel()} scales for {n} output channels")
        scale = scale.contiguous().clone().reshape(n, 1)
        with torch.no_grad():
            scale.mul_(127.0)  # scale -> absmax, what the kernels take (x_pc_max / w_pc_max convention)
        tile_int8_weights_(w_nk)  # in place, marks the tensor; shapes that do not tile stay row-major
        w_1nk = w_nk.view(1, n, k)  # what the grouped GEMM takes; the tiling mark lives on the tensor object
        w_1nk._kmoe_tiled = is_tiled(w_nk)
        layer._kmoe_w_1nk = w_1nk
        setattr(layer, w_q_name, torch.nn.Parameter(w_nk.t(), requires_grad=False))
        setattr(layer, w_s_name, torch.nn.Parameter(scale, requires_grad=False))
        if getattr(layer, i_s_name, None) is not None and not self.config.is_static_input_scheme:
            setattr(layer, i_s_name, None)
        for name in (i_zp_name, azp_adj_name):
            if not hasattr(layer, name):
                setattr(layer, name, None)

    def apply_weights(self, layer: torch.nn.Module, x: torch.Tensor,
                      bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Reference: scale_mm.py:52-90. The symmetric dynamic branch: quantise per token, multiply,
        rescale by x_max * w_max / 127^2, in x's dtype. Output [..., n]."""
        w_q, w_s, x_s, x_zp, azp_adj = self._get_layer_params(layer)
        if azp_adj is not None or x_zp is not None:
            raise NotImplementedError("KunlunScaledMMLinearKernel: asymmetric activations are not implemented")
        if x_s is not None:
            raise NotImplementedError("KunlunScaledMMLinearKernel: static input scales are not implemented")
        if bias is not None:
            raise NotImplementedError("KunlunScaledMMLinearKernel: bias is not implemented on this path")
        if x.dtype != torch.bfloat16:
            raise NotImplementedError(f"KunlunScaledMMLinearKernel: activations must be bf16, got {x.dtype}")
        w = getattr(layer, "_kmoe_w_1nk", None)
        if w is None:
            raise RuntimeError("KunlunScaledMMLinearKernel: process_weights_after_loading has not run on this layer")
        from ...ops import _custom_ops as ops  # registers torch.ops._C.*
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1]).contiguous()
        M, n = x2.shape[0], w.shape[1]
        out = torch.empty((M, n), dtype=x.dtype, device=x.device)
        if M:
            x_q, x_max, _, _ = torch.ops._C.scaled_int8_quant(x2, None, None, True)
            key = (x.device, M)
            if key not in self._lod:
                self._lod[key] = torch.tensor([0, M], dtype=torch.int32).to(x.device)
            ops._gemm_i8(x_q, x_max, w, w_s.data.reshape(-1), self._lod[key], out, n, L.KMOE_ACT_NONE, M)
        return out.reshape(*lead, n)
