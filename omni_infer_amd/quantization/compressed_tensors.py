"""Quantisation config: which method a layer gets.

Mirror of ``AscendCompressedTensorsConfig.get_quant_method``
(omni/quantization/compressed_tensors/compressed_tensors.py:246-262): a ``FusedMoE`` layer gets
the W8A8 MoE method (and ``num_bits`` is set on it), a linear layer gets the W8A8 dynamic
per-token linear scheme; layers named in ``ignore`` (the gate) stay unquantised.  Only the
W8A8 dynamic-token int8 scheme (:81-96, :230-244) is built; anything else raises
NotImplementedError as the reference does for unknown schemes (:61, :139).
"""
from __future__ import annotations

from typing import Iterable, Optional

import torch

from .compressed_tensors_moe import AscendCompressedTensorsW8A8Int8MoEMethod
from .compressed_tensors_w8a8_int8 import AscendCompressedTensorsW8A8Int8LinearMethod

QUANT_NAME = "ascend_compressed_tensors"


class AscendCompressedTensorsConfig:
    def __init__(self, num_bits: int = 8, strategy: str = "channel", dynamic: bool = True,
                 ignore: Optional[Iterable[str]] = None):
        if num_bits != 8:
            raise NotImplementedError("only 8-bit weights / activations are built (W4A8 is an empty stub upstream too)")
        if strategy != "channel" or not dynamic:
            raise NotImplementedError("only per-channel weights with dynamic per-token activations are built")
        self.num_bits = num_bits
        self.strategy = strategy
        self.dynamic = dynamic
        self.ignore = list(ignore or [])

    @classmethod
    def get_name(cls) -> str:
        return QUANT_NAME

    def get_quant_method(self, layer: torch.nn.Module, prefix: str):
        from ..layers.layer import FusedMoE
        from ..layers.linear import ReplicatedLinear
        if any(prefix == ig or prefix.split(".")[-1] == ig for ig in self.ignore):
            return None
        if isinstance(layer, FusedMoE):
            layer.num_bits = self.num_bits
            return AscendCompressedTensorsW8A8Int8MoEMethod()
        if isinstance(layer, ReplicatedLinear):
            return AscendCompressedTensorsW8A8Int8LinearMethod(self.strategy, False, True)
        return None


def register() -> bool:
    """Register the config under the reference's name when vLLM is importable
    (compressed_tensors.py:40, omni/adaptors/vllm/utils.py:44); a no-op otherwise."""
    try:
        from vllm.model_executor.layers.quantization import register_quantization_config  # type: ignore
    except Exception:
        return False
    register_quantization_config(QUANT_NAME)(AscendCompressedTensorsConfig)
    return True
