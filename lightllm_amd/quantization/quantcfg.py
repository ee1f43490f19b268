"""Per-layer resolution of the quantization method for the block-FP8 path.

Mirrors the contract of LightLLM's ``Quantcfg`` (lightllm/common/quantization/__init__.py:21-130): the same
constructor arguments, ``get_quant_type(layer_num, name)`` and ``get_quant_method(layer_num, name)``, the same
precedence between the sources.  Only the block-FP8 method exists in this package, so every source that names an
FP8 128x128-block scheme resolves to it and anything else is refused when it is asked for.

Sources, strongest first, for a given (layer, weight name):
  1. ``expert_dtype`` start argument          - forces the ``fused_moe`` entry of every layer
  2. the YAML file ``custom_cfg_path``         - ``quant_type`` (global) and ``mix_bits`` (per layer / per name)
  3. ``expert_dtype`` in the model config      - fills ``fused_moe`` where the YAML file did not
  4. ``quantization_config`` of the model (HF) - ``quant_method: fp8`` with ``weight_block_size: [128, 128]``
     replaces the global type; the checkpoint then holds quantized weights (``quantized_weight``)
  5. the ``quant_type`` start argument
"""
import collections
from typing import Optional

import yaml

from .registry import QUANTMETHODS

BLOCK_FP8 = "fp8w8a8-b128-mi355"

# what an expert_dtype maps to (reference: EXPERT_DTYPE_TO_QUANT_TYPE, __init__.py:14-18; fp4 needs hardware and
# kernels this package does not have)
EXPERT_DTYPE_TO_QUANT_TYPE = {"fp8": BLOCK_FP8}
SUPPORTED_EXPERT_DTYPES = tuple(EXPERT_DTYPE_TO_QUANT_TYPE)


class Quantcfg:
    def __init__(self, network_config, quant_type="none", custom_cfg_path=None, expert_dtype=None):
        self.layer_num = network_config["n_layer"]
        self.quant_type = quant_type
        self.start_args_expert_dtype = expert_dtype
        self.config_expert_dtype = network_config.get("expert_dtype", None)
        self.quant_cfg = collections.defaultdict(dict)          # layer -> {weight name -> quant type}
        self.hf_quantization_config: Optional[dict] = network_config.get("quantization_config", None)
        self.quantized_weight = self.hf_quantization_config is not None
        self.static_activation = (
            self.quantized_weight and network_config.get("activation_scheme", "dynamic") == "static"
        )
        self.hf_quantization_method = self.hf_quantization_config["quant_method"] if self.quantized_weight else None

        self._read_custom_cfg(custom_cfg_path)                   # source 2 (may replace the global type)
        if self.quantized_weight:
            self._apply_hf_config()                              # source 4
        if not self.quantized_weight or self.hf_quantization_method == "fp8":
            self._apply_expert_dtype()                           # sources 1 and 3

    # ---- sources
    def _read_custom_cfg(self, path):
        if path is None:
            return
        with open(path, "r") as f:
            data = yaml.safe_load(f)
        self.quant_type = data["quant_type"]
        for entry in data.get("mix_bits", []):
            layers = entry.get("layer_nums", range(self.layer_num))
            for layer in layers:
                self.quant_cfg[layer][entry["name"]] = entry["quant_type"]

    def _apply_hf_config(self):
        if self.hf_quantization_method != "fp8":
            return  # other checkpoint formats (awq, ...) keep whatever type was asked for; get_quant_method refuses it
        if self.hf_quantization_config.get("weight_block_size", None) == [128, 128]:
            self.quant_type = BLOCK_FP8

    def _apply_expert_dtype(self):
        dtype = self.start_args_expert_dtype or self.config_expert_dtype
        if dtype is None:
            return
        target = EXPERT_DTYPE_TO_QUANT_TYPE.get(dtype)
        if target is None:
            raise ValueError(f"unsupported expert_dtype `{dtype}`; expected one of {list(SUPPORTED_EXPERT_DTYPES)}")
        forced = self.start_args_expert_dtype is not None
        for layer in range(self.layer_num):
            if forced or "fused_moe" not in self.quant_cfg[layer]:
                self.quant_cfg[layer]["fused_moe"] = target

    # ---- queries
    def get_quant_type(self, layer_num, name):
        per_layer = self.quant_cfg.get(layer_num, None)
        if per_layer is None:
            return self.quant_type
        return per_layer.get(name, self.quant_type)

    def get_quant_method(self, layer_num, name):
        method = QUANTMETHODS.get(self.get_quant_type(layer_num, name))
        method.hf_quantization_config = self.hf_quantization_config
        return method
