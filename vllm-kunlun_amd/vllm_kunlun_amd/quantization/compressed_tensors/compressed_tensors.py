"""The part of vLLM's CompressedTensorsConfig that the MoE method selection needs.

`KunlunCompressedTensorsMoEMethod.get_moe_method(quant_config, layer, layer_name)`
(reference: compressed_tensors_moe.py:43-108) asks the config for the scheme of the three
projections of expert 0. This class answers from the `quantization_config` block of a
checkpoint's config.json (format shown in
docs/source/tutorials/multi_xpu_DeepSeek-V3.2-Exp-w8a8.md:50-95): `config_groups` with
`targets`, `weights`, `input_activations`, `format`; and the `ignore` list.
"""
from __future__ import annotations

import re
from typing import Any, Optional


class CompressedTensorsConfig:
    def __init__(self, target_scheme_map: dict[str, dict[str, Any]], ignore: list[str], quant_format: str = ""):
        self.target_scheme_map = target_scheme_map
        self.ignore = list(ignore)
        self.quant_format = quant_format

    @classmethod
    def from_config(cls, config: dict[str, Any]) -> "CompressedTensorsConfig":
        if config.get("quant_method", "compressed-tensors") != "compressed-tensors":
            raise ValueError(f"not a compressed-tensors checkpoint: quant_method={config.get('quant_method')}")
        targets: dict[str, dict[str, Any]] = {}
        for group in (config.get("config_groups") or {}).values():
            scheme = {"weights": group.get("weights"), "input_activations": group.get("input_activations"),
                      "format": group.get("format", config.get("format"))}
            for target in group.get("targets", []):
                targets[target] = scheme
        return cls(targets, config.get("ignore") or [], config.get("format", ""))

    def get_name(self) -> str:
        return "compressed-tensors"

    def _add_fused_moe_to_target_scheme_map(self) -> None:
        """A FusedMoE is made of Linears: let a scheme that targets Linear reach it."""
        if "Linear" in self.target_scheme_map and "FusedMoE" not in self.target_scheme_map:
            self.target_scheme_map["FusedMoE"] = self.target_scheme_map["Linear"]

    def _ignored(self, layer_name: str) -> bool:
        for pat in self.ignore:
            if pat.startswith("re:"):
                if re.match(pat[3:], layer_name):
                    return True
            elif layer_name == pat or layer_name.endswith("." + pat) or layer_name.startswith(pat + "."):
                return True
        return False

    def get_scheme_dict(self, layer, layer_name: Optional[str] = None) -> Optional[dict[str, Any]]:
        """The scheme of one (unfused) Linear by name; None for an ignored layer."""
        if layer_name is not None and self._ignored(layer_name):
            return None
        for target, scheme in self.target_scheme_map.items():
            if target.startswith("re:"):
                if layer_name is not None and re.match(target[3:], layer_name):
                    return scheme
            elif target in ("Linear", "FusedMoE", type(layer).__name__):
                return scheme
            elif layer_name is not None and (layer_name == target or layer_name.endswith("." + target)):
                return scheme
        return None


class UnquantizedLinearMethod:
    """Named result of get_quant_method for a Linear that the checkpoint leaves unquantized (an
    ignored layer such as lm_head). vLLM's own class of this name serves such layers; a dense bf16
    Linear is not part of the MoE path this package builds, so this stand-in only carries the name."""

    def apply(self, layer, x, bias=None):
        raise NotImplementedError("an unquantized Linear is served by vLLM's UnquantizedLinearMethod, not by this package")


class KunlunCompressedTensorsW8A8Int8LinearMethod:
    """What get_quant_method hands a Linear with a dynamic-token W8A8 int8 scheme: vLLM's
    CompressedTensorsLinearMethod + its CompressedTensorsW8A8Int8 scheme end in the kernel class
    KunlunScaledMMLinearKernel (reference: quantization/kernels/scale_mm.py:30-90); this method is
    that chain in one piece: int8 weight [n, k] + one f32 scale per output channel, loaded by name,
    then process_weights_after_loading / apply of the kernel class."""

    def __init__(self, quant_config: "CompressedTensorsConfig"):
        from ..kernels.scale_mm import Int8ScaledMMLinearLayerConfig, KunlunScaledMMLinearKernel
        self.quant_config = quant_config
        self.kernel = KunlunScaledMMLinearKernel(Int8ScaledMMLinearLayerConfig(
            is_channelwise=True, is_static_input_scheme=False, input_symmetric=True))

    def create_weights(self, layer, input_size_per_partition: int, output_partition_sizes, input_size=None,
                       output_size=None, params_dtype=None, device=None, **_) -> None:
        import torch
        n = int(sum(output_partition_sizes))
        layer.weight = torch.nn.Parameter(torch.zeros(n, input_size_per_partition, dtype=torch.int8, device=device),
                                          requires_grad=False)
        layer.weight_scale = torch.nn.Parameter(torch.zeros(n, 1, dtype=torch.float32, device=device),
                                                requires_grad=False)
        layer.input_scale = None

    def process_weights_after_loading(self, layer) -> None:
        self.kernel.process_weights_after_loading(layer)

    def apply(self, layer, x, bias=None):
        return self.kernel.apply_weights(layer, x, bias)


def _is_linear(layer) -> bool:
    """vLLM's LinearBase subclasses (ColumnParallelLinear, RowParallelLinear, ...), torch's Linear, or any
    stand-in that says so; vLLM is not a dependency, so the test is by class name along the MRO."""
    return any(c.__name__ in ("LinearBase", "Linear") for c in type(layer).__mro__)


def _is_fused_moe(layer) -> bool:
    return any(c.__name__ == "FusedMoE" for c in type(layer).__mro__)


class KunlunCompressedTensorsConfig(CompressedTensorsConfig):
    """The quantization config vLLM asks for every layer's method
    (reference: quantization/compressed_tensors/compressed_tensors.py:47-82, registered there under the
    name "compressed-tensors"). Dispatch on the kind of layer, as the reference does:
      * a FusedMoE       -> KunlunCompressedTensorsMoEMethod.get_moe_method (reference :80-81);
      * a Linear         -> its scheme's method: dynamic-token W8A8 int8 ends in
                            KunlunScaledMMLinearKernel; no scheme (ignored layer) -> unquantized
                            (reference :55-75; transforms and other schemes belong to vLLM's own classes
                            and are refused here by name);
      * Attention (KV-cache scales, reference :77-78) and anything else -> None: outside the MoE path."""

    def get_quant_method(self, layer, prefix: str):
        if _is_fused_moe(layer):
            from .compressed_tensors_moe import KunlunCompressedTensorsMoEMethod
            return KunlunCompressedTensorsMoEMethod.get_moe_method(self, layer, prefix)
        if _is_linear(layer):
            scheme = self.get_scheme_dict(layer, prefix)
            if scheme is None:
                return UnquantizedLinearMethod()
            from .compressed_tensors_moe import _scheme_is_dynamic_token_w8a8
            weight_quant, input_quant = scheme.get("weights"), scheme.get("input_activations")
            if _scheme_is_dynamic_token_w8a8(weight_quant, input_quant):
                layer.scheme = scheme
                return KunlunCompressedTensorsW8A8Int8LinearMethod(self)
            raise NotImplementedError(f"Linear scheme outside this package's path: {weight_quant}, {input_quant}")
        return None


def register_with_vllm() -> None:
    """The two registrations the reference makes at import time, for a process that has vLLM:
    the quantization config under "compressed-tensors" in place of vLLM's own
    (reference: compressed_tensors.py:43-48, quantization/utils.py:22-24) and the unquantized MoE
    method as the out-of-tree implementation of vLLM's CustomOp of that name
    (reference: ops/fused_moe/layer.py:16). Raises ImportError where vLLM is not installed."""
    from vllm.model_executor.custom_op import CustomOp
    from vllm.model_executor.layers.quantization import QUANTIZATION_METHODS, register_quantization_config

    from ...ops.fused_moe.layer import KunlunUnquantizedFusedMoEMethod
    if "compressed-tensors" in QUANTIZATION_METHODS:
        QUANTIZATION_METHODS.remove("compressed-tensors")
    register_quantization_config("compressed-tensors")(KunlunCompressedTensorsConfig)
    CustomOp.register_oot(name="UnquantizedFusedMoEMethod")(KunlunUnquantizedFusedMoEMethod)
