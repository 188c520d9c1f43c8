"""``FusedMoE``: the routed-expert layer of the MoE block on gfx950.

Mirror of omni/models/common/layers/moe/fused_moe/layer.py:169-532: constructor arguments
(:179-199), ``select_experts`` (:301-365), ``apply_expert_load_balance`` (:273-299),
``forward`` (:384-408) and ``weight_loader`` (:410-532) keep their names, argument order and
error behaviour.  vLLM's loader helpers are restated (w1 fills the first half of w13, w3 the
second half; per-channel scales arrive as [out, 1]).
"""
from __future__ import annotations

from typing import Callable, Optional

import os

import torch

from .. import hip_ops as ops
from ..config import model_extra_config
from ..distributed import get_ep_group
from .fused_moe import fused_topk, grouped_topk

UNQUANT_MODE = 0
STATIC_QUANT_MODE = 1
DYNAMIC_QUANT_MODE = 2


class FusedMoE(torch.nn.Module):
    def __init__(self, num_experts: int, top_k: int, hidden_size: int, intermediate_size: int,
                 params_dtype: Optional[torch.dtype] = None, reduce_results: bool = False, renormalize: bool = True,
                 use_grouped_topk: bool = False, num_expert_group: Optional[int] = None,
                 topk_group: Optional[int] = None, quant_config=None, tp_size: Optional[int] = None, prefix: str = "",
                 custom_routing_function: Optional[Callable] = None, scoring_func: str = "softmax",
                 e_score_correction_bias: Optional[torch.Tensor] = None, first_k_dense_replace: int = 3, **kwargs):
        super().__init__()
        self.planner = kwargs.get("planner", None)
        self.moe_layer_idx = kwargs.get("moe_layer_idx", None)
        self.expert_mapping = kwargs.get("expert_mapping", None)
        if model_extra_config.operator_opt_config.enable_moe_expert_parallel:
            ep_size = get_ep_group().world_size - model_extra_config.parall_config.redundancy_shared_expert_num
            num_experts = int(num_experts / ep_size)
            tp_size = 1
        if params_dtype is None:
            params_dtype = torch.get_default_dtype()
        self.tp_size = tp_size if tp_size is not None else get_ep_group().world_size
        self.top_k = top_k
        self.num_experts = num_experts
        self.hidden_size = hidden_size
        self.intermediate_size_per_partition = intermediate_size // self.tp_size
        self.reduce_results = reduce_results
        self.renormalize = renormalize
        self.use_grouped_topk = use_grouped_topk
        if self.use_grouped_topk:
            if num_expert_group is None or topk_group is None:
                raise RuntimeError("num_expert_group and topk_group must not be None")
        self.num_expert_group = num_expert_group
        self.topk_group = topk_group
        self.custom_routing_function = custom_routing_function
        self.is_prefill_instance = os.environ.get("ROLE", "") == "prefill"   # layer.py:228
        if quant_config is None:
            raise NotImplementedError("only the W8A8 quantised MoE method is built (no bf16 expert path)")
        self.quant_method = quant_config.get_quant_method(self, prefix)
        self.quant_mode = DYNAMIC_QUANT_MODE
        if self.quant_method is None:
            raise RuntimeError("self.quant_method must not be None")
        # layer.py:240-246: a rank that deploys redundant copies holds that many more experts
        num_of_redundant_experts = 0
        if model_extra_config.operator_opt_config.use_omni_placement and self.planner is not None:
            num_of_redundant_experts = self.planner.get_num_of_redundant_experts(
                moe_layer_idx=self.moe_layer_idx, num_expert_per_device_origin=num_experts,
                rank_device=get_ep_group().rank_in_group - model_extra_config.parall_config.redundancy_shared_expert_num)
        self.quant_method.create_weights(layer=self, num_experts=num_experts + num_of_redundant_experts, hidden_size=hidden_size,
                                         intermediate_size_per_partition=self.intermediate_size_per_partition,
                                         params_dtype=params_dtype, weight_loader=self.weight_loader,
                                         **({"device": kwargs["device"]} if "device" in kwargs else {}))
        self.scoring_func = scoring_func
        self.e_score_correction_bias = e_score_correction_bias
        if self.scoring_func != "softmax" and not self.use_grouped_topk:
            raise ValueError("Only softmax scoring function is supported for non-grouped topk.")

    def apply_expert_load_balance(self, topk_ids: torch.Tensor, best_topk_ids: Optional[torch.Tensor] = None):
        """layer.py:273-299: the placement planner's remap of the ids to deployed positions when a planner was
        given, then the forced balance of the ``best_ep`` flag: a prefill instance (``ROLE=prefill``) replaces the routing by
        the ids 0..255 dealt round robin, eight per token (the reference hard-codes 256 experts and top-8 at
        :291-292); elsewhere the caller's ``best_topk_ids`` are taken when given."""
        if self.planner is not None:
            _, topk_ids, _ = self.planner.plan(layer_idx_moe=self.moe_layer_idx, tokens=None, token_expert_ids=topk_ids,
                                               token_expert_scores=None, expert_mapping=self.expert_mapping)
        if model_extra_config.operator_opt_config.best_ep:
            if self.is_prefill_instance:
                t = (topk_ids.shape[0] * 8) // 256
                topk_ids = torch.arange(256, device=topk_ids.device, dtype=torch.int32).unsqueeze(0).repeat(t + 1, 1) \
                    .view(-1, 8)[:topk_ids.shape[0]]
            elif best_topk_ids is not None:
                topk_ids = best_topk_ids
        return topk_ids

    @staticmethod
    def select_experts(hidden_states: torch.Tensor, router_logits: torch.Tensor, top_k: int, use_grouped_topk: bool,
                       renormalize: bool, topk_group: Optional[int] = None, num_expert_group: Optional[int] = None,
                       custom_routing_function: Optional[Callable] = None, scoring_func: str = "softmax",
                       e_score_correction_bias: Optional[torch.Tensor] = None,
                       routed_scaling_factor: Optional[float] = None, layer: torch.nn.Module = None):
        """layer.py:301-365, same dispatch: grouped + bias -> the sigmoid/top2-sum router operator;
        grouped without bias -> ``grouped_topk`` times the scaling factor; else ``fused_topk``."""
        if use_grouped_topk:
            if topk_group is None:
                raise ValueError("Unsupported topk_group is None")
            if num_expert_group is None:
                raise ValueError("Unsupported num_expert_group is None")
            if e_score_correction_bias is None:
                topk_weights, topk_ids, row_idx = grouped_topk(
                    hidden_states=hidden_states, gating_output=router_logits, topk=top_k, renormalize=renormalize,
                    num_expert_group=num_expert_group, topk_group=topk_group, scoring_func=scoring_func,
                    e_score_correction_bias=e_score_correction_bias)
                topk_weights = topk_weights * routed_scaling_factor
            else:
                topk_weights, topk_ids, _ = ops.npu_moe_gating_top_k(
                    router_logits.float(), k=top_k, bias=e_score_correction_bias, k_group=topk_group,
                    group_count=num_expert_group, group_select_mode=1, renorm=0, norm_type=1,
                    routed_scaling_factor=routed_scaling_factor, eps=float(1e-20))
                row_idx = ops._row_idx(router_logits.shape[0], top_k, router_logits.device)
        elif custom_routing_function is None:
            topk_weights, topk_ids, row_idx = fused_topk(gating_output=router_logits, topk=top_k,
                                                         renormalize=renormalize)
        else:
            topk_weights, topk_ids, row_idx = custom_routing_function(
                hidden_states=hidden_states, gating_output=router_logits, topk=top_k, renormalize=renormalize)
        return topk_weights, topk_ids, row_idx

    @staticmethod
    def builtin_routing_arguments(top_k: int, use_grouped_topk: bool, renormalize: bool, topk_group: Optional[int],
                                  num_expert_group: Optional[int], custom_routing_function: Optional[Callable],
                                  scoring_func: str, e_score_correction_bias: Optional[torch.Tensor],
                                  routed_scaling_factor: Optional[float]):
        """The arguments the library's router takes for the routing ``select_experts`` (layer.py:301-365) would do,
        scaling factor included, as keywords of ``hip_ops.moe_w8a8_block`` / ``moe_w8a8_layer_routed``; None for
        a custom routing function (which only Python can call)."""
        L = ops.L
        if custom_routing_function is not None and not use_grouped_topk:
            return None
        if use_grouped_topk:
            if topk_group is None:
                raise ValueError("Unsupported topk_group is None")
            if num_expert_group is None:
                raise ValueError("Unsupported num_expert_group is None")
            if e_score_correction_bias is None:
                if scoring_func not in ("softmax", "sigmoid"):
                    raise ValueError(f"Unsupported scoring function: {scoring_func}")
                # grouped_topk (fused_moe.py:38-84) times the scaling factor (layer.py:339): the router's last
                # operation is that multiplication
                return dict(bias=None, top_k=top_k, n_group=num_expert_group, topk_group=topk_group, score_fn=scoring_func,
                            group_mode=L.OMNI_GROUP_MAX, masked_fill_zero=True, weight_from_c=True,
                            renorm=bool(renormalize), scale=float(routed_scaling_factor), eps=0.0)
            # npu_moe_gating_top_k as called at layer.py:341-351
            return dict(bias=e_score_correction_bias, top_k=top_k, n_group=num_expert_group, topk_group=topk_group,
                        score_fn="sigmoid", group_mode=L.OMNI_GROUP_TOP2SUM, masked_fill_zero=False, weight_from_c=False,
                        renorm=True, scale=float(routed_scaling_factor), eps=float(1e-20))
        # fused_topk (fused_moe.py:24-34)
        return dict(bias=None, top_k=top_k, n_group=1, topk_group=1, score_fn="softmax", group_mode=L.OMNI_GROUP_MAX,
                    masked_fill_zero=False, weight_from_c=False, renorm=bool(renormalize), scale=1.0, eps=0.0)

    @staticmethod
    def gate_and_select_experts(hidden_states: torch.Tensor, gate_weight: torch.Tensor, top_k: int,
                                use_grouped_topk: bool, renormalize: bool, topk_group: Optional[int] = None,
                                num_expert_group: Optional[int] = None,
                                custom_routing_function: Optional[Callable] = None, scoring_func: str = "softmax",
                                e_score_correction_bias: Optional[torch.Tensor] = None,
                                routed_scaling_factor: Optional[float] = None, want_logits: bool = False):
        """``gate.forward(hidden_states.float())`` followed by ``select_experts`` (deepseek_moe.py:253-256,
        329-333) as one library call: the tokens are read as they are (no fp32 copy), the logits are summed
        in the library's fixed order and routed by the same three routers with the same arguments as
        ``select_experts`` gives them.  Returns (topk_weights, topk_ids, row_idx, router_logits or None)."""
        L = ops.L
        bf16_gate = gate_weight.dtype == torch.bfloat16
        T = hidden_states.shape[0]
        if use_grouped_topk:
            if topk_group is None:
                raise ValueError("Unsupported topk_group is None")
            if num_expert_group is None:
                raise ValueError("Unsupported num_expert_group is None")
            if e_score_correction_bias is None:
                if scoring_func not in ("softmax", "sigmoid"):
                    raise ValueError(f"Unsupported scoring function: {scoring_func}")
                # grouped_topk (fused_moe.py:38-84), then the scaling factor (layer.py:339)
                w, ids, logits = ops.moe_gate_route(hidden_states, gate_weight, None, top_k, num_expert_group, topk_group,
                                                    scoring_func, L.OMNI_GROUP_MAX, True, True, bool(renormalize), 1.0,
                                                    0.0, want_logits, bf16_gate)
                w = w * routed_scaling_factor
            else:
                # npu_moe_gating_top_k as called at layer.py:341-351
                w, ids, logits = ops.moe_gate_route(hidden_states, gate_weight, e_score_correction_bias, top_k,
                                                    num_expert_group, topk_group, "sigmoid", L.OMNI_GROUP_TOP2SUM, False,
                                                    False, True, routed_scaling_factor, float(1e-20), want_logits,
                                                    bf16_gate)
        elif custom_routing_function is None:
            # fused_topk (fused_moe.py:24-34)
            w, ids, logits = ops.moe_gate_route(hidden_states, gate_weight, None, top_k, 1, 1, "softmax",
                                                L.OMNI_GROUP_MAX, False, False, bool(renormalize), 1.0, 0.0, want_logits,
                                                bf16_gate)
        else:
            logits = ops.gate_logits(hidden_states, gate_weight, round_logits_bf16=bf16_gate)
            w, ids, row_idx = custom_routing_function(hidden_states=hidden_states, gating_output=logits, topk=top_k,
                                                      renormalize=renormalize)
            return w, ids, row_idx, logits
        return w, ids, ops._row_idx(T, top_k, hidden_states.device), logits

    def forward(self, hidden_states: torch.Tensor, topk_weights: torch.Tensor, topk_ids: torch.Tensor,
                pertoken_scale: torch.Tensor, attn_metadata, comm_group=None):
        """layer.py:384-408 (the all-reduce of a tensor-parallel expert split is not built:
        one GPU)."""
        if self.quant_method is None:
            raise RuntimeError("self.quant_method must not be None")
        return self.quant_method.apply(layer=self, x=hidden_states, topk_weights=topk_weights, topk_ids=topk_ids,
                                       pertoken_scale=pertoken_scale, attn_metadata=attn_metadata,
                                       comm_group=comm_group)

    # ------------------------------------------------------------------ checkpoint loading
    def _local_expert(self, expert_id: int) -> int:
        """Global -> local expert id, -1 if another rank owns it (layer.py:414-430); with a placement the pattern
        says whether the rank deploys the expert and at which local position (:417-424)."""
        if not model_extra_config.operator_opt_config.enable_moe_expert_parallel:
            return expert_id
        if model_extra_config.operator_opt_config.use_omni_placement and self.planner is not None:
            ep_rank = get_ep_group().rank_in_group - model_extra_config.parall_config.redundancy_shared_expert_num
            exists_locally, local_pos = self.planner.is_expert_on_current_rank(self.moe_layer_idx, expert_id, ep_rank,
                                                                               self.num_experts)
            return local_pos if exists_locally else -1
        lo = get_ep_group().rank_in_group * self.num_experts
        return expert_id - lo if lo <= expert_id < lo + self.num_experts else -1

    def weight_loader(self, param: torch.nn.Parameter, loaded_weight: torch.Tensor, weight_name: str, shard_id: str,
                      expert_id: int) -> None:
        """layer.py:410-532 for the per-channel int8 format: ``shard_id`` is w1 (gate), w3 (up)
        or w2 (down); weights are [out, in], scales/offsets [out, 1]."""
        if shard_id not in ("w1", "w2", "w3"):
            raise ValueError(f"shard_id must be ['w1','w2','w3'] but got {shard_id}.")
        local = self._local_expert(expert_id)
        if local < 0:
            return
        I = self.intermediate_size_per_partition
        data = param.data[local]
        if "scale" in weight_name or "offset" in weight_name:
            loaded_weight = loaded_weight.squeeze(-1)  # [out, 1] -> [out]   (layer.py:372)
        loaded_weight = loaded_weight.to(data.device)
        if shard_id == "w2":
            data.copy_(loaded_weight)
        elif shard_id == "w1":
            data[:I].copy_(loaded_weight)
        else:
            data[I:2 * I].copy_(loaded_weight)
