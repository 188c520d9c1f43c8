"""W8A8 int8 MoE quantisation method on gfx950.

Mirror of omni/quantization/compressed_tensors/compressed_tensors_moe.py:
``AscendCompressedTensorsW8A8Int8MoEMethod.{create_weights, process_weights_after_loading,
apply}`` (:26-219) and ``fused_experts_w8a8`` (:221-254), same signatures.  The branches of
``apply`` that need a process group (all-to-all dispatch/combine across ranks) are computed
in their one-rank form: with a single rank the dispatch is the local sort by expert and the
combine is the local weighted un-permute.
"""
from __future__ import annotations

import os
from typing import Optional

import torch

from .. import _lib as L
from .. import hip_ops as ops
from ..config import model_extra_config
from ..distributed import get_ep_group
from ..layers.fused_moe import (fused_experts_w8a8_allgather_ep, fused_experts_w8a8_allgather_ep_a2,
                                moe_expert_quant_farword)

SEQ_SPLIT_LENGTH = 4096


def set_weight_attrs(weight: torch.Tensor, attrs: Optional[dict]) -> None:
    """vllm.model_executor.utils.set_weight_attrs: attach loader attributes to a parameter."""
    if not attrs:
        return
    for k, v in attrs.items():
        setattr(weight, k, v)


class AscendCompressedTensorsW8A8Int8MoEMethod:
    def __init__(self):
        self.initialized = False
        self.warm_up = True
        self.n_routed_experts = None
        self.smooth_scale = None

    def create_weights(self, layer: torch.nn.Module, num_experts: int, hidden_size: int,
                       intermediate_size_per_partition: int, params_dtype: torch.dtype, **extra_weight_attrs) -> None:
        """compressed_tensors_moe.py:34-92: checkpoint-layout parameters.  w13 int8 [E, 2I, H]
        (w1/gate rows then w3/up rows), w2 int8 [E, H, I], per-channel scales and offsets
        [E, 2I] / [E, H] in bf16 (fp32 when the model dtype is fp16)."""
        dev = extra_weight_attrs.pop("device", None)
        sdt = torch.float32 if params_dtype == torch.float16 else torch.bfloat16
        I = intermediate_size_per_partition

        def param(t):
            return torch.nn.Parameter(t, requires_grad=False)

        w13 = param(torch.empty(num_experts, 2 * I, hidden_size, dtype=torch.int8, device=dev))
        layer.register_parameter("w13_weight", w13)
        set_weight_attrs(w13, extra_weight_attrs)
        w2 = param(torch.empty(num_experts, hidden_size, I, dtype=torch.int8, device=dev))
        layer.register_parameter("w2_weight", w2)
        set_weight_attrs(w2, extra_weight_attrs)
        extra_weight_attrs.update({"quant_method": "channel"})
        for name, shape, fill in (("w13_weight_scale", (num_experts, 2 * I), 1.0),
                                  ("w13_weight_offset", (num_experts, 2 * I), 0.0),
                                  ("w2_weight_scale", (num_experts, hidden_size), 1.0),
                                  ("w2_weight_offset", (num_experts, hidden_size), 0.0)):
            p = param(torch.full(shape, fill, dtype=sdt, device=dev))
            layer.register_parameter(name, p)
            set_weight_attrs(p, extra_weight_attrs)
        layer.hidden_size = hidden_size
        layer.intermediate_size_per_partition = I

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        """compressed_tensors_moe.py:94-114.  The reference transposes the weights to
        [E, H, 2I] / [E, I, H] and optionally casts them to its matrix-unit format; here the
        checkpoint layout goes straight into the frag16 layout of the gfx950 kernels (one
        pass, the transpose is implied).  Scale dtypes follow the reference's flags."""
        opt = model_extra_config.operator_opt_config
        layer.w13_weight = torch.nn.Parameter(ops.pack_weight(layer.w13_weight.data, 1), requires_grad=False)
        layer.w2_weight = torch.nn.Parameter(ops.pack_weight(layer.w2_weight.data, 1), requires_grad=False)
        if opt.pd_seperate_prefill:
            layer.w2_weight_scale = torch.nn.Parameter(layer.w2_weight_scale.to(torch.bfloat16), requires_grad=False)
        elif not opt.opt_w2_scale_cast:
            layer.w2_weight_scale = torch.nn.Parameter(layer.w2_weight_scale.to(torch.float32), requires_grad=False)
        layer.w13_weight_scale = torch.nn.Parameter(layer.w13_weight_scale.to(torch.float32).contiguous(),
                                                    requires_grad=False)
        self.n_routed_experts = len(layer.w13_weight)
        self.local_expert_indices_offset = get_ep_group().rank_in_group * self.n_routed_experts
        self.local_expert_indices = [self.local_expert_indices_offset + i for i in range(self.n_routed_experts)]
        self.initialized = True
        self.smooth_scale = torch.ones((self.n_routed_experts, layer.w13_weight_scale.shape[-1] // 2),
                                       dtype=torch.float32, device=layer.w13_weight.device)

    def apply(self, layer: torch.nn.Module, x: torch.Tensor, topk_weights: torch.Tensor, topk_ids: torch.Tensor,
              pertoken_scale: torch.Tensor, attn_metadata, comm_group=None) -> torch.Tensor:
        """compressed_tensors_moe.py:116-219, same branch conditions."""
        opt = model_extra_config.operator_opt_config
        n_local = self.n_routed_experts
        max_num_deployed_expert_per_rank = n_local   # :126-128
        planner = getattr(layer, "planner", None)
        if opt.use_omni_placement and planner is not None and planner.is_moe_layer(layer.moe_layer_idx):
            max_num_deployed_expert_per_rank = planner.get_max_num_deployed_expert_per_rank()
        if opt.enable_moe_expert_parallel:
            is_prefill = attn_metadata is None or attn_metadata.prefill is not None
            if opt.prefill_dispatch_combine or (opt.moe_dispatch_combine and not is_prefill):
                if get_ep_group().world_size != 1:
                    raise NotImplementedError(
                        "dispatch/combine across ranks needs collectives; this build runs one GPU. "
                        "Use the all-gather expert-parallel flags (prefill_dispatch_combine=False, "
                        "moe_dispatch_combine=False) for one GPU's share of a larger model.")
                out = fused_experts_w8a8_one_rank_dispatch_combine(layer, x, topk_weights, topk_ids)
            elif os.getenv("ASCEND_PLATFORM", "A3") == "A2":   # the reference's own switch (:157)
                out = fused_experts_w8a8_allgather_ep_a2(
                    hidden_states=x, pertoken_scale=pertoken_scale, w1=layer.w13_weight, w2=layer.w2_weight,
                    w1_scale=layer.w13_weight_scale, w2_scale=layer.w2_weight_scale, topk_weights=topk_weights,
                    topk_ids=topk_ids, n_routed_experts=n_local, is_prefill=is_prefill,
                    max_num_deployed_expert_per_rank=max_num_deployed_expert_per_rank, smooth_scale=self.smooth_scale)
            else:
                out = fused_experts_w8a8_allgather_ep(
                    hidden_states=x, pertoken_scale=pertoken_scale, w1=layer.w13_weight, w2=layer.w2_weight,
                    w1_scale=layer.w13_weight_scale, w2_scale=layer.w2_weight_scale, topk_weights=topk_weights,
                    topk_ids=topk_ids, n_routed_experts=n_local, is_prefill=is_prefill,
                    max_num_deployed_expert_per_rank=max_num_deployed_expert_per_rank)
            if self.warm_up:
                self.warm_up = False
            return out
        token_num = x.shape[0]
        if token_num > SEQ_SPLIT_LENGTH:  # split the sequence to bound the scratch memory (:190-209)
            outs = []
            for xs, ws, ids in zip(x.split(SEQ_SPLIT_LENGTH), topk_weights.split(SEQ_SPLIT_LENGTH),
                                   topk_ids.split(SEQ_SPLIT_LENGTH)):
                outs.append(fused_experts_w8a8(xs, layer.w13_weight, layer.w2_weight, layer.w13_weight_scale,
                                               layer.w2_weight_scale, layer.w13_weight_offset, layer.w2_weight_offset,
                                               ws, ids, ops._row_idx(xs.shape[0], ids.shape[1], x.device)))
            return torch.concat(outs)
        return fused_experts_w8a8(x, layer.w13_weight, layer.w2_weight, layer.w13_weight_scale, layer.w2_weight_scale,
                                  layer.w13_weight_offset, layer.w2_weight_offset, topk_weights, topk_ids,
                                  ops._row_idx(token_num, topk_ids.shape[1], x.device))


def fused_experts_w8a8(hidden_states: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, w1_scale: torch.Tensor,
                       w2_scale: torch.Tensor, w1_offset, w2_offset, topk_weights: torch.Tensor,
                       topk_ids: torch.Tensor, row_idx: torch.Tensor) -> torch.Tensor:
    """compressed_tensors_moe.py:221-254: the non-EP pipeline.  bf16 tokens are sorted by
    expert (k*T+n numbering), quantised, pushed through GEMM1 with a bf16 dequant, SwiGLU in
    bf16, requantised, GEMM2 with bf16 rows, and combined in ascending k.  The weight scales
    are rounded to bf16 first (:239-240)."""
    T, H = hidden_states.shape
    E = len(w1)
    K = topk_ids.shape[1]
    I = w1_scale.shape[-1] // 2
    p = ops.moe_permute(topk_ids, 0, E, L.OMNI_IDX_K_MAJOR)
    x_q, x_s = ops.npu_dynamic_quant(hidden_states)  # per token; sorting rows first gives the same rows
    s1 = w1_scale.to(torch.bfloat16).float().contiguous()
    s2 = w2_scale.to(torch.bfloat16).float().contiguous()
    h_q, h_s, _ = ops.grouped_gemm1_swiglu_quant(x_q, x_s, p.sorted_src, L.OMNI_IDX_K_MAJOR, K, w1, s1, p.offsets, H, I,
                                                 T * K, bf16_intermediate=True)
    rows, _ = ops.grouped_gemm2_dequant(h_q, h_s, w2, s2, p.offsets, H, I, out_dtype=torch.bfloat16)
    return ops.moe_combine(rows, topk_weights, p.src_to_dst, L.OMNI_IDX_K_MAJOR, L.OMNI_ORDER_K)


def fused_experts_w8a8_one_rank_dispatch_combine(layer, x: torch.Tensor, topk_weights: torch.Tensor,
                                                 topk_ids: torch.Tensor) -> torch.Tensor:
    """One-rank form of ``fused_experts_w8a8_moe_dispatch_combine`` (fused_moe.py:690-791):
    quantise and sort the tokens by expert (what the dispatch operator hands to a rank),
    run ``moe_expert_quant_farword`` on the grouped rows, and weight the bf16 rows back per
    token in ascending k (what the combine operator returns)."""
    T, H = x.shape
    E = len(layer.w13_weight)
    p = ops.moe_permute(topk_ids, 0, E, L.OMNI_IDX_TOKEN_MAJOR)
    if x.dtype != torch.int8:
        x_q, x_s = ops.npu_dynamic_quant(x)
    else:
        raise ValueError("dispatch/combine takes unquantised tokens")
    rows_q, rows_s = ops.moe_gather_rows(x_q, x_s, p)
    planner = getattr(layer, "planner", None)
    if model_extra_config.operator_opt_config.use_omni_placement and planner is not None:
        planner.record_activation(layer.moe_layer_idx, p.counts, True)   # fused_moe.py:745-746
    rows = moe_expert_quant_farword(rows_q, layer.w13_weight, layer.w2_weight, layer.w13_weight_scale,
                                    layer.w2_weight_scale, p.counts, torch.bfloat16, 2, rows_s)
    return ops.moe_combine(rows, topk_weights, p.src_to_dst, L.OMNI_IDX_TOKEN_MAJOR, L.OMNI_ORDER_K)


class AscendCompressedTensorsW4A8Int8MoEMethod:
    """Declared and left empty by the reference as well (compressed_tensors_moe.py:256-257)."""
    pass
