"""Quantisation config: which method a layer gets, read from the checkpoint's own description.

Mirror of ``AscendCompressedTensorsConfig`` (omni/quantization/compressed_tensors/compressed_tensors.py:40-264):
``get_config_filenames`` (:63-65: the checkpoint directory holds ``quant_model_description.json``),
``from_config`` (:183-222: one entry per target of every config group, the weights' ``num_bits`` kept as it
is written, a number or a per-module dict), ``_get_weight_num_bits`` (:67-78), ``_is_dynamic_token_w8a8`` /
``_is_dynamic_token_w4a8`` (:81-114), ``_get_scheme_from_parts`` (:117-139), ``get_scheme`` (:142-180),
``get_moe_method`` (:230-244) and ``get_quant_method`` (:246-262).  The pieces of vLLM and of the
``compressed_tensors`` package the reference leans on are restated here in a few lines each (neither is
installed in this image): ``QuantArgs`` stands for ``QuantizationArgs`` (only the fields the selection reads),
``find_matched_target`` and ``should_ignore_layer`` for the functions of the same names in vLLM's
``compressed_tensors/utils.py``.

Only the W8A8 dynamic per-token int8 scheme is built; W4A8 (empty stubs upstream) and anything else raise
NotImplementedError / RuntimeError where the reference does (:139, :243).
"""
from __future__ import annotations

import json
import os
import re
from dataclasses import dataclass
from typing import Any, Dict, Iterable, List, Optional, Union

import torch

from .compressed_tensors_moe import AscendCompressedTensorsW4A8Int8MoEMethod, AscendCompressedTensorsW8A8Int8MoEMethod
from .compressed_tensors_w8a8_int8 import AscendCompressedTensorsW8A8Int8LinearMethod

QUANT_NAME = "ascend_compressed_tensors"

# compressed_tensors.config.CompressionFormat values whose activations are quantised
# (vLLM: is_activation_quantization_format)
ACTIVATION_QUANTIZATION_FORMATS = ("naive-quantized", "int-quantized", "float-quantized", "nvfp4-pack-quantized")


@dataclass
class QuantArgs:
    """The fields of ``compressed_tensors.quantization.QuantizationArgs`` the scheme selection reads, with that
    model's defaults.  ``num_bits`` of a weight entry may be a dict {module name part: bits} (:67-78)."""
    num_bits: Union[int, Dict[str, int]] = 8
    type: str = "int"
    symmetric: bool = True
    group_size: Optional[int] = None
    strategy: Optional[str] = None
    dynamic: bool = False

    @classmethod
    def parse_obj(cls, obj: Dict[str, Any]) -> "QuantArgs":
        if not isinstance(obj, dict):
            raise ValueError(f"quantization arguments must be a mapping, got {type(obj).__name__}")
        known = {k: obj[k] for k in ("num_bits", "type", "symmetric", "group_size", "strategy", "dynamic") if k in obj}
        args = cls(**known)
        if args.strategy is None:   # QuantizationArgs derives the strategy from the group size when it is not given
            args.strategy = "tensor" if args.group_size in (None, -1) else "group"
        args.strategy = str(args.strategy).lower()
        return args


def _is_equal_or_regex_match(value: str, target: str, check_contains: bool = False) -> bool:
    if target.startswith("re:"):
        return re.match(target[3:], value) is not None
    if check_contains:
        return target.lower() in value.lower()
    return target == value


def find_matched_target(layer_name: Optional[str], module: torch.nn.Module, targets: Iterable[str]) -> str:
    """The target of the config a layer conforms to: its full name, a ``re:`` pattern on its name, or a part of
    its class name ("Linear" matches ``ReplicatedLinear``), in that order."""
    layer_name = layer_name or ""
    targets = list(targets)
    for t in targets:
        if _is_equal_or_regex_match(layer_name, t):
            return t
    for t in targets:
        if _is_equal_or_regex_match(module.__class__.__name__, t, check_contains=True):
            return t
    raise ValueError(f"Unable to find matching target for {layer_name} in the compressed-tensors config.")


def should_ignore_layer(layer_name: Optional[str], ignore: Iterable[str]) -> bool:
    """A layer stays unquantised when the ``ignore`` list names it: by its full name, by a ``re:`` pattern, or by
    its last name component (``gate``, ``lm_head``)."""
    if layer_name is None:
        return False
    for ig in ignore:
        if _is_equal_or_regex_match(layer_name, ig) or layer_name.split(".")[-1] == ig:
            return True
    return False


class AscendCompressedTensorsConfig:
    quant_description: Dict[str, Any] = {}

    def __init__(self, target_scheme_map: Optional[Dict[str, Any]] = None, ignore: Optional[Iterable[str]] = None,
                 quant_format: str = "int-quantized", kv_cache_scheme: Optional[Dict[str, Any]] = None,
                 sparsity_scheme_map=None, sparsity_ignore_list=None, *, num_bits: int = 8, strategy: str = "channel",
                 dynamic: bool = True):
        """As the reference's parent class is constructed by ``from_config`` (:217-222).  Without a
        ``target_scheme_map`` the keyword-only arguments describe the one scheme this build runs (8-bit
        per-channel weights, dynamic per-token activations) for every ``Linear``."""
        if target_scheme_map is None:
            target_scheme_map = {"Linear": {
                "weights": QuantArgs(num_bits=num_bits, strategy=strategy, dynamic=False, symmetric=True),
                "input_activations": QuantArgs(num_bits=num_bits, strategy="token", dynamic=bool(dynamic), symmetric=True)}}
            # this constructor form promises the built scheme: refuse anything else here rather than at a layer
            self.target_scheme_map, self.quant_format = target_scheme_map, quant_format
            self._get_scheme_from_parts("", target_scheme_map["Linear"]["weights"],
                                        target_scheme_map["Linear"]["input_activations"])
            if strategy != "channel":
                raise NotImplementedError("only per-channel weights with dynamic per-token activations are built")
        self.target_scheme_map = target_scheme_map
        self.ignore = list(ignore or [])
        self.quant_format = quant_format
        self.kv_cache_scheme = kv_cache_scheme
        self.sparsity_scheme_map = sparsity_scheme_map
        self.sparsity_ignore_list = sparsity_ignore_list

    def __repr__(self) -> str:
        return f"AscendCompressedTensorsConfig:\n  targets={list(self.target_scheme_map)} ignore={self.ignore} format={self.quant_format}"

    @classmethod
    def get_name(cls) -> str:
        return QUANT_NAME

    @classmethod
    def get_supported_act_dtypes(cls) -> List[torch.dtype]:
        return [torch.int8, torch.float16, torch.bfloat16]

    @classmethod
    def get_min_capability(cls) -> int:
        raise NotImplementedError("Ascend hardware dose not support \"get_min_capability\" feature.")

    @classmethod
    def get_config_filenames(cls) -> List[str]:
        return ["quant_model_description.json"]

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_config(cls, config: Dict[str, Any]) -> "AscendCompressedTensorsConfig":
        """compressed_tensors.py:183-222."""
        cls.quant_description = config
        target_scheme_map: Dict[str, Any] = {}
        ignore = config.get("ignore")
        quant_format = config.get("format")
        for _, group in config["config_groups"].items():
            for target in group.get("targets"):
                entry: Dict[str, Any] = {}
                # the per-module num_bits dict is kept as written, not validated (:202-207)
                entry["weights"] = QuantArgs.parse_obj(group.get("weights"))
                try:
                    entry["input_activations"] = QuantArgs.parse_obj(group.get("input_activations"))
                except Exception:
                    entry["input_activations"] = None
                target_scheme_map[target] = entry
        return cls(target_scheme_map=target_scheme_map, ignore=ignore, quant_format=quant_format,
                   kv_cache_scheme=config.get("kv_cache_scheme"), sparsity_scheme_map=None, sparsity_ignore_list=None)

    @classmethod
    def from_checkpoint_dir(cls, path: str) -> "AscendCompressedTensorsConfig":
        """What vLLM's loader does with ``get_config_filenames``: the first of those files found in the
        checkpoint directory is parsed as JSON and handed to ``from_config``."""
        for name in cls.get_config_filenames():
            f = os.path.join(path, name)
            if os.path.isfile(f):
                with open(f) as fh:
                    return cls.from_config(json.load(fh))
        raise ValueError(f"Cannot find the config file for {QUANT_NAME} in {path}: expected one of "
                         f"{cls.get_config_filenames()}")

    # ------------------------------------------------------------------ scheme selection
    def _get_weight_num_bits(self, layer_name: str, weight_quant: QuantArgs):
        """:67-78."""
        if isinstance(weight_quant.num_bits, dict):
            for module, module_num_bits in weight_quant.num_bits.items():
                if module in layer_name:
                    return module_num_bits
            raise ValueError("weight name mismatch, please check weights num_bits in config.json and model weight "
                             f"name. layer_name={layer_name}")
        return weight_quant.num_bits

    @staticmethod
    def _weight_strategy_ok(weight_quant: QuantArgs) -> bool:
        return weight_quant.strategy in ("tensor", "channel", "group")

    def _is_dynamic_token_w8a8(self, weight_quant: QuantArgs, input_quant: Optional[QuantArgs], weight_num_bits) -> bool:
        """:81-96: symmetric static 8-bit weights (per tensor, channel or group), dynamic per-token 8-bit inputs."""
        if input_quant is None:
            return False
        is_8_bits = weight_num_bits == input_quant.num_bits == 8
        is_token = self._weight_strategy_ok(weight_quant) and input_quant.strategy == "token"
        is_dynamic = not weight_quant.dynamic and input_quant.dynamic
        return bool(is_8_bits and is_token and weight_quant.symmetric and is_dynamic)

    def _is_dynamic_token_w4a8(self, weight_quant: QuantArgs, input_quant: Optional[QuantArgs], weight_num_bits) -> bool:
        """:99-114."""
        if input_quant is None:
            return False
        is_w4a8_bits = weight_num_bits == 4 and input_quant.num_bits == 8
        is_token = self._weight_strategy_ok(weight_quant) and input_quant.strategy == "token"
        is_dynamic = not weight_quant.dynamic and input_quant.dynamic
        return bool(is_w4a8_bits and is_token and weight_quant.symmetric and is_dynamic)

    def _get_scheme_from_parts(self, layer_name: str, weight_quant: QuantArgs, input_quant: Optional[QuantArgs]):
        """:117-139."""
        if self.quant_format in ACTIVATION_QUANTIZATION_FORMATS:
            weight_num_bits = self._get_weight_num_bits(layer_name, weight_quant)
            if self._is_dynamic_token_w8a8(weight_quant, input_quant, weight_num_bits):
                return AscendCompressedTensorsW8A8Int8LinearMethod(strategy=weight_quant.strategy,
                                                                   is_static_input_scheme=False,
                                                                   input_symmetric=input_quant.symmetric)
            if self._is_dynamic_token_w4a8(weight_quant, input_quant, weight_num_bits):
                # the reference returns its W4A8 linear scheme here; its kernels are not part of this build
                raise NotImplementedError("the W4A8 scheme is not built (only W8A8 dynamic per-token int8 is)")
        raise NotImplementedError("No compressed-tensors compatible scheme was found.")

    def get_scheme(self, layer: torch.nn.Module, layer_name: Optional[str] = None):
        """:142-180."""
        matched_target = find_matched_target(layer_name=layer_name, module=layer, targets=self.target_scheme_map.keys())
        scheme_dict = self.target_scheme_map[matched_target]
        return self._get_scheme_from_parts(layer_name=layer_name or "", weight_quant=scheme_dict["weights"],
                                           input_quant=scheme_dict["input_activations"])

    def get_moe_method(self, prefix: str):
        """:230-244: the routed experts take the scheme of the ``Linear`` target, their bit width the entry of
        ``mlp.experts`` in a per-module ``num_bits``."""
        weight_quant = self.target_scheme_map["Linear"].get("weights")
        input_quant = self.target_scheme_map["Linear"].get("input_activations")
        weight_num_bits = self._get_weight_num_bits("mlp.experts", weight_quant)
        if self._is_dynamic_token_w8a8(weight_quant, input_quant, weight_num_bits):
            return AscendCompressedTensorsW8A8Int8MoEMethod(), weight_num_bits
        if self._is_dynamic_token_w4a8(weight_quant, input_quant, weight_num_bits):
            return AscendCompressedTensorsW4A8Int8MoEMethod(), weight_num_bits
        raise RuntimeError(f"Unsupported FusedMoe scheme: {weight_quant}, {input_quant}")

    def get_quant_method(self, layer: torch.nn.Module, prefix: str):
        """:246-262.  A layer the ``ignore`` list names stays unquantised (None), as the parent class of the
        reference's config decides before anything else."""
        from ..layers.layer import FusedMoE
        from ..layers.linear import ReplicatedLinear
        if should_ignore_layer(prefix, self.ignore):
            return None
        if isinstance(layer, ReplicatedLinear):
            scheme = self.get_scheme(layer=layer, layer_name=prefix)
            layer.scheme = scheme
            return scheme
        if isinstance(layer, FusedMoE):
            layer.num_bits = 0
            moe_method, weight_num_bits = self.get_moe_method(prefix)
            layer.num_bits = weight_num_bits
            return moe_method
        return None

    def get_scaled_act_names(self) -> List[str]:
        return []


def register() -> bool:
    """Register the config under the reference's name when vLLM is importable
    (compressed_tensors.py:40, omni/adaptors/vllm/utils.py:44); a no-op otherwise."""
    try:
        from vllm.model_executor.layers.quantization import register_quantization_config  # type: ignore
    except Exception:
        return False
    register_quantization_config(QUANT_NAME)(AscendCompressedTensorsConfig)
    return True
