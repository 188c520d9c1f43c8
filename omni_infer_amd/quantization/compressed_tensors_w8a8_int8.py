"""W8A8 int8 dense linear scheme (the shared expert's projections) on gfx950.

Mirror of omni/quantization/compressed_tensors/schemes/compressed_tensors_w8a8_int8.py:
``AscendCompressedTensorsW8A8Int8LinearMethod.{create_weights, process_weights_after_loading,
apply_weights}`` (:19-110), channel strategy with dynamic per-token activations.
"""
from __future__ import annotations

from typing import Any, Callable, Dict, List, Optional, Union

import torch
from torch.nn import Parameter

from .. import hip_ops as ops

BEFORE_INIT = 0
AFTER_INIT = 1


class AscendCompressedTensorsW8A8Int8LinearMethod:
    def __init__(self, strategy: str = "channel", is_static_input_scheme: bool = False, input_symmetric: bool = True):
        if strategy != "channel" or is_static_input_scheme:
            raise NotImplementedError("only per-channel weights with dynamic per-token activations are built")
        self.strategy = strategy
        self.is_static_input_scheme = is_static_input_scheme
        self.input_symmetric = input_symmetric

    def create_weights(self, layer: torch.nn.Module, output_partition_sizes: List[int], input_size_per_partition: int,
                       params_dtype: torch.dtype, weight_loader: Optional[Callable] = None, **kwargs):
        """w8a8_int8.py:33-69: weight int8 [out, in]; weight_scale / weight_offset [out, 1]."""
        dev = kwargs.get("device", None)
        out = sum(output_partition_sizes)
        sdt = torch.float32 if params_dtype == torch.float16 else torch.bfloat16
        self.logical_widths = output_partition_sizes
        layer.register_parameter("weight", Parameter(torch.empty(out, input_size_per_partition, dtype=torch.int8,
                                                                 device=dev), requires_grad=False))
        layer.register_parameter("weight_scale", Parameter(torch.empty(out, 1, dtype=sdt, device=dev),
                                                           requires_grad=False))
        layer.register_parameter("weight_offset", Parameter(torch.zeros(out, 1, dtype=sdt, device=dev),
                                                            requires_grad=False))
        layer.input_size_per_partition = input_size_per_partition
        layer.output_size = out
        setattr(layer, "init_state", BEFORE_INIT)

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        """w8a8_int8.py:73-84: the reference transposes to [in, out] and casts to its matrix
        format; here [out, in] is packed into the frag16 layout.  Scales are flattened; they are
        widened to fp32 for the kernels (the reference widens when ``throw_dequant`` is set,
        otherwise its operator widens internally)."""
        layer.weight = Parameter(ops.pack_weight(layer.weight.data, 1), requires_grad=False)
        layer.weight_scale = Parameter(layer.weight_scale.data.view(-1).float().contiguous(), requires_grad=False)
        layer.weight_offset = Parameter(layer.weight_offset.data.view(-1).float(), requires_grad=False)

    def apply_weights(self, layer: torch.nn.Module, x: Union[torch.Tensor, Dict[str, Any]],
                      bias: Optional[torch.Tensor]) -> Union[torch.Tensor, Dict[str, Any], tuple]:
        """w8a8_int8.py:86-110.  A layer marked ``throw_dequant`` hands back the quantised input
        and its scale together with itself, so that the following ``SiluAndMul`` runs GEMM +
        dequant + SwiGLU + requant as one fused operator (the reference returns the raw int32
        product there, :99-103; the int32 matrix never leaves the chip here)."""
        if layer.init_state == BEFORE_INIT:
            layer.init_state = AFTER_INIT
        if isinstance(x, Dict):
            x_int8, pertoken_scale = x.get("x_int8"), x.get("pertoken_scale")
        else:
            x_int8, pertoken_scale = ops.npu_dynamic_quant(x)
        if bias is not None:
            raise NotImplementedError("bias is not used on the MoE path")
        if getattr(layer, "throw_dequant", False):
            return (DeferredInt32Matmul(x_int8, layer), pertoken_scale)
        M = x_int8.shape[0]
        offsets = ops.dense_offsets(M, x_int8.device)
        rows, _ = ops.grouped_gemm2_dequant(x_int8.contiguous(), pertoken_scale.contiguous(), layer.weight,
                                            layer.weight_scale, offsets, layer.output_size,
                                            layer.input_size_per_partition, out_dtype=torch.bfloat16)
        return rows


class DeferredInt32Matmul:
    """The int8 input of a GEMM whose int32 result is consumed by the fused SwiGLU operator."""

    def __init__(self, x_int8: torch.Tensor, layer: torch.nn.Module):
        self.x_int8 = x_int8
        self.layer = layer

    @property
    def shape(self):
        return (self.x_int8.shape[0], self.layer.output_size)
