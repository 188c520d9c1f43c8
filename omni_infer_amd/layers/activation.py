"""``SiluAndMul`` of the quantised path (omni/models/common/layers/activation.py:10-29)."""
from __future__ import annotations

from typing import Any, Dict, Union

import torch
import torch.nn as nn

from .. import hip_ops as ops
from ..quantization.compressed_tensors_w8a8_int8 import DeferredInt32Matmul


class SiluAndMul(nn.Module):
    def forward(self, x: Union[Dict[str, Any], torch.Tensor], quant_symbol: bool = False):
        """Quantised input (a dict with ``x_int8``, ``pertoken_scale``, ``out_scale``): the fused
        dequant + SwiGLU + requant (activation.py:15-28), returning ``{x_int8, pertoken_scale}``.
        A plain bf16 tensor: SwiGLU in fp32 rounded once to bf16 (``npu_swiglu``, :29) -- that
        branch is outside the W8A8 path and is not built."""
        if quant_symbol and isinstance(x, Dict):
            src = x.get("x_int8")
            if not isinstance(src, DeferredInt32Matmul):
                raise ValueError("SiluAndMul expects the deferred int32 product of a throw_dequant linear")
            layer = src.layer
            H, I = layer.input_size_per_partition, layer.output_size // 2
            M = src.x_int8.shape[0]
            offsets = ops.dense_offsets(M, src.x_int8.device)
            h, s, _ = ops.grouped_gemm1_swiglu_quant(src.x_int8.contiguous(), x.get("pertoken_scale").contiguous(),
                                                     None, 0, 1, layer.weight, x.get("out_scale").float().contiguous(),
                                                     offsets, H, I, M)
            return {"x_int8": h, "pertoken_scale": s}
        raise NotImplementedError("only the W8A8 path is built (bf16 SwiGLU is outside it)")
