"""Dense W8A8 linear layer (the shared expert's gate_up and down projections, and any other
int8 Linear of a W8A8 checkpoint).

Mirror of `KunlunScaledMMLinearKernel` (reference: quantization/kernels/scale_mm.py:30-90), which
vLLM's `CompressedTensorsW8A8Int8` scheme instantiates per Linear. The reference derives from
vLLM's `CutlassInt8ScaledMMLinearKernel`; vLLM is not a dependency here, so this class carries the
few pieces of that base it relies on (the parameter names and what the base's
`process_weights_after_loading` leaves behind: the weight as the [k, n] transpose view of its
[n, k] storage, a per-channel weight scale, no input scale for dynamic quantisation).

Path taken by `apply_weights`: per-token absmax int8 quantisation and the grouped int8 GEMM
(`kmoe_grouped_gemm_i8`) on the weights re-arranged at load time into the MFMA tiles - for up to 256
rows as the tail expert of the weight-streaming kernel, beyond as its one-expert case on the tile
kernel: the same kernels the fused MoE layer runs its shared expert on.
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
        front which schemes its kernels cover: all four (dynamic or static input scale, symmetric or
        asymmetric activations)."""
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
        # Static input scheme (base-class part, upstream vLLM's CutlassInt8ScaledMMLinearKernel, which is not in
        # this container: restated from its published source): a layer fused from several checkpoint tensors
        # (qkv, gate_up) carries one input scale - and zero point - per partition, and the kernels take ONE.
        # Symmetric: the largest scale. Asymmetric: the value range every partition covers,
        # [min_p scale_p (-128 - zp_p), max_p scale_p (127 - zp_p)], cut into 255 steps again.
        if self.config.is_static_input_scheme:
            i_s = getattr(layer, i_s_name, None)
            if i_s is None:
                raise ValueError(f"{i_s_name}: a static input scheme needs the input scale")
            s_in = i_s.data.to(torch.float32).reshape(-1)
            if self.config.input_symmetric:
                setattr(layer, i_s_name, torch.nn.Parameter(s_in.max().reshape(1), requires_grad=False))
            else:
                i_zp = getattr(layer, i_zp_name, None)
                if i_zp is None:
                    raise ValueError(f"{i_zp_name}: a static asymmetric scheme needs the input zero point")
                zps = i_zp.data.to(torch.int32).reshape(-1)
                if zps.numel() not in (1, s_in.numel()):
                    raise ValueError(f"{i_zp_name}: {zps.numel()} zero points for {s_in.numel()} input scales")
                if s_in.numel() > 1:  # (one partition: its scale and zero point are kept as they are)
                    range_max = (s_in * (127 - zps)).max()
                    range_min = (s_in * (-128 - zps)).min()
                    one_scale = (range_max - range_min) / 255.0
                    # rounded to the nearest integer: the quotient is an integer up to float error when one
                    # partition spans the whole range, and truncation would then lose one
                    one_zp = torch.round(-128 - range_min / one_scale).to(torch.int32)
                    setattr(layer, i_s_name, torch.nn.Parameter(one_scale.reshape(1), requires_grad=False))
                    setattr(layer, i_zp_name, torch.nn.Parameter(one_zp.reshape(1), requires_grad=False))
        # Asymmetric activations (base-class part): azp_adj = the sums of the weight codes over k per output channel,
        # times the input zero point for a static scheme, whose zero point then needs no term of its own at run time.
        if not self.config.input_symmetric:
            azp_adj = w_nk.sum(dim=1, dtype=torch.int32).reshape(1, n)
            if self.config.is_static_input_scheme:
                i_zp = getattr(layer, i_zp_name, None)
                if i_zp is None:
                    raise ValueError(f"{i_zp_name}: a static asymmetric scheme needs the input zero point")
                azp_adj = azp_adj * i_zp.data.to(torch.int32).reshape(1, 1)
            setattr(layer, azp_adj_name, torch.nn.Parameter(azp_adj.contiguous(), requires_grad=False))
        tile_int8_weights_(w_nk)  # in place, marks the memory; shapes that do not tile stay row-major
        layer._kmoe_w_1nk = w_nk.view(1, n, k)  # what the grouped GEMM takes
        setattr(layer, w_q_name, torch.nn.Parameter(w_nk.t(), requires_grad=False))
        setattr(layer, w_s_name, torch.nn.Parameter(scale, requires_grad=False))
        if getattr(layer, i_s_name, None) is not None and not self.config.is_static_input_scheme:
            setattr(layer, i_s_name, None)
        for name in (i_zp_name, azp_adj_name):
            if not hasattr(layer, name):
                setattr(layer, name, None)

    def apply_weights(self, layer: torch.nn.Module, x: torch.Tensor,
                      bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Reference: scale_mm.py:52-90. The symmetric branch: quantise per token (dynamic) or with the
        layer's one input scale (static), multiply, rescale by x_max * w_max / 127^2, in x's dtype.
        Output [..., n]."""
        w_q, w_s, x_s, x_zp, azp_adj = self._get_layer_params(layer)
        if azp_adj is not None:
            return self._apply_asymmetric(layer, x, w_q, w_s, x_s, x_zp, azp_adj, bias)
        if bias is not None:
            # the reference's call (scale_mm.py:83-90): quantise, then matmul with the f32 bias
            x2 = x.reshape(-1, x.shape[-1]).contiguous()
            x_q, x_s2, _, static = torch.ops._C.scaled_int8_quant(
                x2, None if x_s is None else x_s.data.to(torch.float32).reshape(1), None, True)
            out = torch.ops._C.matmul(x_q, w_q.transpose(0, 1), x.dtype, x_pc_max=x_s2 * 127.0 if static else x_s2,
                                      w_pc_max=w_s.data, bias=bias.to(torch.float32).contiguous())
            return out.reshape(*x.shape[:-1], out.shape[-1])
        dt = L.act_dtype(x, "KunlunScaledMMLinearKernel")
        w = getattr(layer, "_kmoe_w_1nk", None)
        if w is None:
            raise RuntimeError("KunlunScaledMMLinearKernel: process_weights_after_loading has not run on this layer")
        from ...ops import _custom_ops as ops  # registers torch.ops._C.*
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1]).contiguous()
        M, n, k = x2.shape[0], w.shape[1], w.shape[2]
        out = torch.empty((M, n), dtype=x.dtype, device=x.device)
        if M == 0:
            return out.reshape(*lead, n)
        if x_s is not None:  # static: one scale for the tensor, so every row's max is scale x 127
            x_q, x_s, _, _ = torch.ops._C.scaled_int8_quant(x2, x_s.data.to(torch.float32).reshape(1), None, True)
            x_max = (x_s * 127.0).expand(M).contiguous()
            ops._gemm_i8(x_q, x_max, w, w_s.data.reshape(-1), self._row_range(x.device, M), out, n, L.KMOE_ACT_NONE, M)
        elif is_tiled(w) and M <= self.STREAM_MAX_ROWS:
            self._stream_gemm(x2, w, w_s.data.reshape(-1), out)
        else:
            x_q, x_max, _, _ = torch.ops._C.scaled_int8_quant(x2, None, None, True)
            ops._gemm_i8(x_q, x_max, w, w_s.data.reshape(-1), self._row_range(x.device, M), out, n, L.KMOE_ACT_NONE, M)
        return out.reshape(*lead, n)

    def _apply_asymmetric(self, layer, x, w_q, w_s, x_s, x_zp, azp_adj, bias):
        """Reference: scale_mm.py:60-82. Codes with a zero point (per token, or the layer's static one), the int8
        product, and the zero-point correction in the epilogue; the weight scale goes back from absmax to scale
        (/ 127) as there."""
        L.act_dtype(x, "KunlunScaledMMLinearKernel")
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1]).contiguous()
        x_q, x_s, x_zp, static = torch.ops._C.scaled_int8_quant(
            x2, None if x_s is None else x_s.data.to(torch.float32).reshape(1),
            None if x_zp is None else x_zp.data.to(torch.int32).reshape(1), False)
        out = torch.ops._C.cutlass_scaled_mm_azp(
            x_q, w_q, x_s, (w_s.data / 127.0).transpose(0, 1), x.dtype, azp_adj.data, None if static else x_zp,
            None if bias is None else bias.to(torch.float32).contiguous())
        return out.reshape(*lead, out.shape[-1])

    # Up to this many rows the GEMM runs on the weight-streaming kernel (the one the fused MoE layer
    # runs decode batches and its folded shared expert on): the dense matrix is handed over as the
    # launch's "tail expert", whose rows the kernel cuts into slices of 16 or 32 for as many
    # workgroups - a tile kernel has too few tiles to fill the chip here. Measured on
    # [M,7168] x [4096,7168]: 16 us against 36 us at 16 rows, 25 against 38 at 128, 31 against 38 at 256;
    # at 512 rows the tile kernel is ahead (39 against 46 us).
    STREAM_MAX_ROWS = 256

    def _row_range(self, device, rows):
        key = (device, rows)
        if key not in self._lod:
            self._lod[key] = torch.tensor([0, rows], dtype=torch.int32).to(device)
        return self._lod[key]

    def _stream_gemm(self, x2, w, w_max, out):
        M, k = x2.shape
        n = w.shape[1]
        x_q = torch.empty((k // 64, M, 64), dtype=torch.int8, device=x2.device)  # chunk-major codes
        x_max = torch.empty((M,), dtype=torch.float32, device=x2.device)
        L.check(L.lib.kmoe_quant_i8_rows_chunked_dt(L.ptr(x2), k, M, k, L.ptr(x_q), L.ptr(x_max),
                                                    L.act_dtype(x2), L.stream()))
        g = L.GemmI8Args()
        g.a, g.lda, g.a_max, g.src_div = x_q.data_ptr(), k, x_max.data_ptr(), 1
        g.a_layout, g.a_rows = L.KMOE_A_CHUNKED, M
        # one routed expert without rows (the launch needs an expert list), the matrix as the tail expert
        g.w, g.w_max, g.lod = w.data_ptr(), w_max.data_ptr(), self._row_range(x2.device, 0).data_ptr()
        g.E, g.n, g.k, g.rows = 1, n, k, 0
        g.w_tail, g.w_max_tail = w.data_ptr(), w_max.data_ptr()
        g.tail_row0, g.tail_rows, g.tail_src0 = 0, M, 0
        g.y, g.ldy, g.act, g.w_layout = out.data_ptr(), n, L.KMOE_ACT_NONE, L.KMOE_W_TILED
        g.act_dtype = L.act_dtype(out)
        g.variant = 1 if M <= 128 else 2  # 16 or 32 rows per slice
        L.check(L.lib.kmoe_grouped_gemm_i8(g, L.stream()))
