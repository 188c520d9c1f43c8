"""RMSNorm with the fused residual add and the optional int8 hand-over to the MoE block.

Mirror of ``RMSNorm`` in omni/models/common/layers/layernorm.py:13-32 (a subclass of vLLM's
``RMSNorm``: parameters ``weight`` [hidden_size] in the model dtype and ``variance_epsilon``).
``forward(x, residual, quant_symbol)``:
  * with a residual: returns ``(x, residual)`` where ``x`` is the normalised tensor, or, when
    ``use_w8a8_dynamic_quant`` is on and ``quant_symbol`` is set, the dict
    ``{"x_int8": ..., "pertoken_scale": ...}`` the quantised linear layers and the MoE block accept
    (:21-25);
  * without one: returns the normalised tensor (:28-32).
All of it is one kernel launch here (omni_add_rms_norm_quant).
"""
from __future__ import annotations

from typing import Any, Optional, Union

import torch
import torch.nn as nn

from .. import hip_ops as ops
from ..config import model_extra_config


class RMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float = 1e-6, var_hidden_size: Optional[int] = None,
                 params_dtype: Optional[torch.dtype] = None, device=None):
        super().__init__()
        if var_hidden_size is not None and var_hidden_size != hidden_size:
            raise NotImplementedError("partial-width variance is not used by the models on this path")
        self.hidden_size = hidden_size
        self.variance_epsilon = eps
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=params_dtype or torch.get_default_dtype(),
                                              device=device), requires_grad=False)

    def forward(self, x: torch.Tensor, residual: Optional[torch.Tensor] = None,
                quant_symbol: bool = False) -> Union[tuple[dict[str, Any], Any], Any]:
        if residual is not None:
            quant = bool(model_extra_config.operator_opt_config.use_w8a8_dynamic_quant and quant_symbol)
            y, residual, x_int8, pertoken_scale = ops.add_rms_norm_quant(
                x, residual, self.weight.data, self.variance_epsilon, want_y=not quant, want_quant=quant)
            if quant:
                return {"x_int8": x_int8, "pertoken_scale": pertoken_scale}, residual
            return y, residual
        y, _, _, _ = ops.add_rms_norm_quant(x, None, self.weight.data, self.variance_epsilon)
        return y

    def forward_moe_input(self, x: torch.Tensor, residual: torch.Tensor):
        """Not in the reference: the same launch also emits the int8 rows and per-token scales the
        MoE block would otherwise make with its own quantisation pass (deepseek_moe.py:247,323).
        Returns ``({"x": y, "x_int8": q, "pertoken_scale": s}, residual)``; ``DeepseekMoE.forward``
        accepts the dict in place of the hidden states."""
        y, residual, x_int8, pertoken_scale = ops.add_rms_norm_quant(
            x, residual, self.weight.data, self.variance_epsilon, want_y=True, want_quant=True)
        return {"x": y, "x_int8": x_int8, "pertoken_scale": pertoken_scale}, residual
