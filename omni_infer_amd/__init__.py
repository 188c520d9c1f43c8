"""MI355X-native W8A8 dynamic-quant fused-MoE layer behind omni-infer's MoE interfaces.

Public surface (the reference's names for this path):
  quantization.compressed_tensors.AscendCompressedTensorsConfig
  quantization.compressed_tensors_moe.AscendCompressedTensorsW8A8Int8MoEMethod
  quantization.compressed_tensors_w8a8_int8.AscendCompressedTensorsW8A8Int8LinearMethod
  layers.layer.FusedMoE, layers.deepseek_moe.{DeepseekMoE, ReplicatedDeepseekMLP}
  layers.fused_moe.{fused_topk, grouped_topk, fused_experts_w8a8_allgather_ep, ...}
  hip_ops: the operator boundary over libomni_moe_hip.so (include/omni_moe_hip.h)
"""
__version__ = "0.1.0"
