"""Replicated linear layers used by the MoE block: the gate and the shared expert's projections.

Mirror of ``ReplicatedLinear`` / ``MergedReplicatedLinear`` as the MoE block uses them
(omni/models/common/layers/linear.py:620-762; deepseek_moe.py:74-84,147-152): no tensor
parallelism, ``forward`` returns ``(output, None)``.
"""
from __future__ import annotations

from typing import List, Optional

import torch
import torch.nn as nn


class ReplicatedLinear(nn.Module):
    def __init__(self, input_size: int, output_size: int, bias: bool = False, quant_config=None,
                 params_dtype: Optional[torch.dtype] = None, prefix: str = "", device=None):
        super().__init__()
        if bias:
            raise NotImplementedError("bias is not used on the MoE path")
        self.input_size, self.output_size = input_size, output_size
        self.prefix = prefix
        self.params_dtype = params_dtype or torch.get_default_dtype()
        self.quant_method = quant_config.get_quant_method(self, prefix) if quant_config is not None else None
        if self.quant_method is None:
            self.weight = nn.Parameter(torch.empty(output_size, input_size, dtype=self.params_dtype, device=device),
                                       requires_grad=False)
        else:
            self.quant_method.create_weights(self, [output_size], input_size, self.params_dtype, device=device)

    def forward(self, x):
        if self.quant_method is None:
            if not x.is_cuda:
                raise RuntimeError("omni_infer_amd operators run on the GPU only (got a CPU tensor)")
            if self._gate_shaped(x):
                # the unquantised replicated linear of the MoE path is the gate (deepseek_moe.py:147-152): its
                # product runs on the fp32 matrix cores in the library's fixed summation order; a bf16 gate
                # (deepseek_v3_a2.py:607-613) hands back bf16 logits
                from .. import hip_ops as ops
                lead = x.shape[:-1]
                bf16_gate = self.weight.dtype == torch.bfloat16
                logits = ops.gate_logits(x.reshape(-1, x.shape[-1]), self.weight, round_logits_bf16=bf16_gate)
                if bf16_gate:
                    logits = logits.to(torch.bfloat16)
                return logits.view(*lead, self.output_size), None
            # any other unquantised replicated linear (a projection the checkpoint's ``ignore`` list names, fp16
            # parameters, a width the gate kernel does not take): the plain product of the reference's
            # unquantised linear method, ``F.linear(x, weight)`` (linear.py:620-638)
            return torch.nn.functional.linear(x.to(self.weight.dtype), self.weight), None
        return self.quant_method.apply_weights(self, x, None), None

    def _gate_shaped(self, x) -> bool:
        """What the library's gate projection takes: at most 512 outputs, a reduction length that is a multiple
        of 128, bf16 or fp32 operands."""
        return (self.output_size <= 512 and self.input_size % 128 == 0 and
                x.dtype in (torch.bfloat16, torch.float32) and self.weight.dtype in (torch.bfloat16, torch.float32))

    def weight_loader(self, param: nn.Parameter, loaded_weight: torch.Tensor) -> None:
        """vLLM's ``ReplicatedLinear.weight_loader``: a whole-parameter copy; shapes must agree."""
        if param.data.shape != loaded_weight.shape:
            raise RuntimeError("param_data.shape != loaded_weight.shape")
        param.data.copy_(loaded_weight)


class MergedReplicatedLinear(ReplicatedLinear):
    """gate_proj and up_proj stacked along the output dim (linear.py:620-762)."""

    def __init__(self, input_size: int, output_sizes: List[int], bias: bool = False, quant_config=None,
                 params_dtype: Optional[torch.dtype] = None, prefix: str = "", device=None):
        self.output_sizes = output_sizes
        super().__init__(input_size, sum(output_sizes), bias, quant_config, params_dtype, prefix, device)

    def weight_loader(self, param: nn.Parameter, loaded_weight: torch.Tensor,
                      loaded_shard_id: Optional[int] = None) -> None:
        """linear.py:639-762 for parameters stacked along dim 0 (weights [out, in], per-channel
        scales and offsets [out, 1]): shard ``i`` fills rows ``sum(output_sizes[:i])`` onwards;
        without a shard id a fused checkpoint tensor is split over the shards."""
        if loaded_shard_id is None:
            if param.data.shape[0] != loaded_weight.shape[0]:
                raise RuntimeError("param_data.shape != loaded_weight.shape")
            offset = 0
            for i, size in enumerate(self.output_sizes):
                self.weight_loader(param, loaded_weight.narrow(0, offset, size), i)
                offset += size
            return
        if loaded_shard_id >= len(self.output_sizes):
            raise RuntimeError("loaded_shard_id >= len(self.output_sizes)")
        offset = sum(self.output_sizes[:loaded_shard_id])
        size = self.output_sizes[loaded_shard_id]
        dst = param.data.narrow(0, offset, size)
        src = loaded_weight.narrow(0, 0, size)
        if dst.shape != src.shape:
            raise RuntimeError("param_data.shape != loaded_weight.shape")
        dst.copy_(src)
