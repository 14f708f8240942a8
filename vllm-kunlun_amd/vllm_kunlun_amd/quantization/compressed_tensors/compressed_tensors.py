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
