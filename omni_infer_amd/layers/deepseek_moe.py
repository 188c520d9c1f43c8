"""The MoE block: gate, shared expert, routed experts.

Mirror of omni/models/common/layers/moe/deepseek_moe.py: ``ReplicatedDeepseekMLP`` (:64-118)
and ``DeepseekMoE`` (:121-368) with ``forward(hidden_states, residual, attn_metadata, layer_id,
next_attention_weights=None) -> (hidden_states, residual)`` (:228).  The collectives of the
reference (all_gather before, reduce_scatter after the experts) are not issued: one GPU
computes its own expert share on its own tokens.

``forward`` has two bodies with the same results:
  * the operator-by-operator sequence of the reference (`_forward_norm_ops`), kept for parity
    checks, and
  * the fused sequence (default): one quantisation feeds both the shared expert and the routed
    experts, and the shared expert rides through the two grouped GEMM launches as an extra
    group, so the layer is one library call after the router.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch
from torch import nn

from .. import hip_ops as ops
from ..config import model_extra_config
from ..distributed import get_ep_group, get_world_group
from ..placement import OmniPlanner
from .activation import SiluAndMul
from .layer import FusedMoE
from .linear import MergedReplicatedLinear, ReplicatedLinear

SEQ_SPLIT_LENGTH = 4096


class ReplicatedDeepseekMLP(nn.Module):
    """deepseek_moe.py:64-118."""

    def __init__(self, hidden_size: int, intermediate_size: int, hidden_act: str, quant_config=None,
                 reduce_results: bool = True, prefix: str = "", device=None) -> None:
        super().__init__()
        self.gate_up_proj = MergedReplicatedLinear(hidden_size, [intermediate_size] * 2, bias=False,
                                                   quant_config=quant_config, prefix=f"{prefix}.gate_up_proj",
                                                   device=device)
        self.gate_up_proj.throw_dequant = True
        self.down_proj = ReplicatedLinear(intermediate_size, hidden_size, bias=False, quant_config=quant_config,
                                          prefix=f"{prefix}.down_proj", device=device)
        if hidden_act != "silu":
            raise ValueError(f"Unsupported activation: {hidden_act}. Only silu is supported for now.")
        self.act_fn_obj = SiluAndMul()
        self.quant_symbol = True if quant_config else False

    def act_fn(self, x, quant_symbol):
        if quant_symbol and isinstance(x, tuple):
            x = dict(zip(["x_int8", "pertoken_scale"], x))
            x["out_scale"] = self.gate_up_proj.weight_scale
        return self.act_fn_obj(x, quant_symbol)

    def _one(self, x):
        gate_up, _ = self.gate_up_proj.forward(x)
        x = self.act_fn(gate_up, self.quant_symbol)
        x, _ = self.down_proj.forward(x)
        return x

    def forward(self, x):
        token_num = x.get("x_int8").shape[0] if isinstance(x, Dict) else x.shape[0]
        if token_num > SEQ_SPLIT_LENGTH and not isinstance(x, Dict):  # :105-114
            return torch.concat([self._one(c) for c in x.split(SEQ_SPLIT_LENGTH)])
        return self._one(x)


class DeepseekMoE(nn.Module):
    """deepseek_moe.py:121-368.  ``config`` needs: hidden_size, n_routed_experts,
    num_experts_per_tok, moe_intermediate_size, n_shared_experts, n_group, topk_group,
    norm_topk_prob, scoring_func, topk_method, routed_scaling_factor, hidden_act,
    first_k_dense_replace."""

    def __init__(self, config, quant_config=None, prefix: str = "", device=None, planner=None):
        super().__init__()
        self.prefix = prefix
        self.ep_size = get_ep_group().world_size
        self.routed_scaling_factor = config.routed_scaling_factor
        self.redundancy_shared_expert_num = model_extra_config.parall_config.redundancy_shared_expert_num
        if self.redundancy_shared_expert_num != 0:
            raise NotImplementedError("dedicated shared-expert ranks need a process group; one GPU here")
        self.quant_symbol = quant_config is not None
        if self.ep_size > config.n_routed_experts:
            raise ValueError(f"Tensor parallel size {self.ep_size} is greater than "
                             f"the number of experts {config.n_routed_experts} + 0.")
        if config.hidden_act != "silu":
            raise ValueError(f"Unsupported activation: {config.hidden_act}. Only silu is supported for now.")
        self.gate = ReplicatedLinear(config.hidden_size, config.n_routed_experts, bias=False, quant_config=None,
                                     params_dtype=torch.float32, prefix=f"{prefix}.gate", device=device)
        if config.topk_method == "noaux_tc":
            self.gate.e_score_correction_bias = nn.Parameter(
                torch.empty(config.n_routed_experts, dtype=torch.float, device=device), requires_grad=False)
        else:
            self.gate.e_score_correction_bias = None
        self.global_rank = get_world_group().rank_in_group
        # deepseek_moe.py:161-176: with a placement the routed experts are addressed by deployed position
        self.planner = self.moe_layer_idx = self.expert_mapping = None
        if model_extra_config.operator_opt_config.use_omni_placement:
            self.planner = planner if planner is not None else OmniPlanner(
                config_file=model_extra_config.operator_opt_config.omni_placement_config_path, device=device or "cuda",
                rank=get_world_group().rank_in_group, world_size=get_world_group().world_size,
                num_experts=config.n_routed_experts, num_redundancy_shared_expert_rank=self.redundancy_shared_expert_num)
            self.moe_layer_idx = OmniPlanner.get_deepseek_v3_moe_layer_idx(
                f"{prefix}.experts", getattr(config, "first_k_dense_replace", 3))
            self.expert_mapping = self.planner.expert_mapping_on_current_layer(self.moe_layer_idx)
        self.experts = FusedMoE(
            num_experts=config.n_routed_experts, top_k=config.num_experts_per_tok, hidden_size=config.hidden_size,
            intermediate_size=config.moe_intermediate_size, reduce_results=False, renormalize=config.norm_topk_prob,
            quant_config=quant_config, use_grouped_topk=True, num_expert_group=config.n_group,
            topk_group=config.topk_group, prefix=f"{prefix}.experts", scoring_func=config.scoring_func,
            e_score_correction_bias=self.gate.e_score_correction_bias,
            first_k_dense_replace=getattr(config, "first_k_dense_replace", 3), device=device,
            planner=self.planner, moe_layer_idx=self.moe_layer_idx, expert_mapping=self.expert_mapping)
        self.shared_experts = None
        if config.n_shared_experts is not None:
            self.shared_experts = ReplicatedDeepseekMLP(
                hidden_size=config.hidden_size, intermediate_size=config.moe_intermediate_size * config.n_shared_experts,
                hidden_act=config.hidden_act, quant_config=quant_config, reduce_results=False,
                prefix=f"{prefix}.shared_experts", device=device)
        self.local_expert_num = self.experts.w13_weight.shape[0]
        self.fused = True
        # how the expert rows travel from GEMM2 to the weighted sum in the fused body: fp32 is what the
        # reference's fused GEMM2+finalize operator accumulates from (fused_moe.py:536); torch.bfloat16
        # halves the largest intermediate of a prefill-sized call at the price of one more rounding
        self.rows_dtype = torch.float32
        self._workspace = None

    def process_weights_after_loading(self) -> None:
        """What vLLM's loader does after the checkpoint is in: every quant method re-lays its weights."""
        self.experts.quant_method.process_weights_after_loading(self.experts)
        if self.shared_experts is not None:
            for lin in (self.shared_experts.gate_up_proj, self.shared_experts.down_proj):
                if lin.quant_method is not None:
                    lin.quant_method.process_weights_after_loading(lin)

    def _positions_per_rank(self) -> int:
        """Width of a rank's range of expert ids: its experts, or with a placement the deployed positions every
        rank is given (compressed_tensors_moe.py:126-128; fused_moe.py:510)."""
        if self.planner is not None and self.planner.is_moe_layer(self.moe_layer_idx):
            return self.planner.get_max_num_deployed_expert_per_rank()
        return self.local_expert_num

    def _route(self, hidden_states, attn_metadata=None):
        """``self.gate.forward(hidden_states.float())`` + ``FusedMoE.select_experts`` (deepseek_moe.py:253-256,
        329-333).  The fused body makes both in one library call on the tokens as they are; the
        operator-by-operator body keeps the reference's two steps.  Same bits either way."""
        e = self.experts
        if self.fused:
            topk_weights, topk_ids, _, _ = FusedMoE.gate_and_select_experts(
                hidden_states, self.gate.weight, e.top_k, e.use_grouped_topk, e.renormalize, e.topk_group,
                e.num_expert_group, e.custom_routing_function, e.scoring_func, e.e_score_correction_bias,
                self.routed_scaling_factor)
        else:
            router_logits, _ = self.gate.forward(hidden_states.float())
            topk_weights, topk_ids, _ = FusedMoE.select_experts(
                hidden_states, router_logits, e.top_k, e.use_grouped_topk, e.renormalize, e.topk_group,
                e.num_expert_group, e.custom_routing_function, e.scoring_func, e.e_score_correction_bias,
                self.routed_scaling_factor, layer=e)
        # the decode paths hand the forced-balance ids of the attention metadata on (deepseek_moe.py:343, :399)
        best = getattr(getattr(attn_metadata, "decode", None), "best_topk", None)
        return topk_weights, e.apply_expert_load_balance(topk_ids=topk_ids, best_topk_ids=best)

    def forward(self, hidden_states: torch.Tensor, residual: torch.Tensor, attn_metadata, layer_id: int = 0,
                next_attention_weights: Optional[dict] = None):
        opt = model_extra_config.operator_opt_config
        allgather_ep = opt.enable_moe_expert_parallel and self.ep_size > 1 and not (
            opt.prefill_dispatch_combine or opt.moe_dispatch_combine)
        same_width = (self.shared_experts is None or
                      self.shared_experts.down_proj.input_size == self.experts.intermediate_size_per_partition)
        if self.fused and allgather_ep and same_width and self.quant_symbol:
            return self._forward_fused(hidden_states, attn_metadata), residual
        if isinstance(hidden_states, dict):
            hidden_states = hidden_states["x"]
        return self._forward_norm_ops(hidden_states, attn_metadata), residual

    def _forward_norm_ops(self, hidden_states, attn_metadata):
        """deepseek_moe.py:243-305 / :307-368 operator by operator, minus the collectives."""
        opt = model_extra_config.operator_opt_config
        shared_output = self.shared_experts(hidden_states) if self.shared_experts is not None else None
        is_prefill = attn_metadata is None or attn_metadata.prefill is not None
        dispatch = opt.prefill_dispatch_combine if is_prefill else opt.moe_dispatch_combine
        if not dispatch and opt.enable_moe_expert_parallel:
            x_in, pertoken_scale = ops.npu_dynamic_quant(hidden_states)
        else:
            x_in, pertoken_scale = hidden_states, None
        topk_weights, topk_ids = self._route(hidden_states, attn_metadata)
        final = self.experts(hidden_states=x_in, topk_weights=topk_weights, topk_ids=topk_ids,
                             pertoken_scale=pertoken_scale, attn_metadata=attn_metadata)
        if shared_output is not None:
            final = final + shared_output
        return final

    def _forward_fused(self, hidden_states, attn_metadata=None):
        # a dict from RMSNorm.forward_moe_input carries the tokens already quantised
        x_int8 = pertoken_scale = None
        if isinstance(hidden_states, dict):
            x_int8, pertoken_scale = hidden_states["x_int8"], hidden_states["pertoken_scale"]
            hidden_states = hidden_states["x"]
        e = self.experts
        lo = self.global_rank * self._positions_per_rank()
        shared = None
        if self.shared_experts is not None:
            gu, dn = self.shared_experts.gate_up_proj, self.shared_experts.down_proj
            shared = (gu.weight, gu.weight_scale, dn.weight, dn.weight_scale)
        T, K = hidden_states.shape[0], e.top_k
        E = self.gate.weight.shape[0]
        need = ops.L.lib().omni_moe_w8a8_block_workspace_bytes(T, K, self.local_expert_num, e.hidden_size,
                                                               e.intermediate_size_per_partition, E,
                                                               int(shared is not None), ops._DT[self.rows_dtype])
        if self._workspace is None or self._workspace.numel() < need:
            self._workspace = torch.empty(need, dtype=torch.uint8, device=hidden_states.device)
        # The ids the router makes go straight into the experts unless something has to see them first: the
        # placement planner's remap, the forced balance of best_ep (layer.py:273-299), a routing function only
        # Python can call, or tokens the library cannot quantise itself.  Then the block is one library call:
        # gate projection, router, quantisation, sort, both GEMMs, weighted sum.
        opt = model_extra_config.operator_opt_config
        routing = FusedMoE.builtin_routing_arguments(
            e.top_k, e.use_grouped_topk, e.renormalize, e.topk_group, e.num_expert_group, e.custom_routing_function,
            e.scoring_func, e.e_score_correction_bias, self.routed_scaling_factor)
        one_call = (routing is not None and e.planner is None and not opt.best_ep and e.hidden_size % 128 == 0 and
                    (x_int8 is not None or hidden_states.dtype == torch.bfloat16) and
                    hidden_states.dtype in (torch.bfloat16, torch.float32))
        if one_call:
            out, _, _ = ops.moe_w8a8_block(hidden_states, self.gate.weight, lo=lo, hi=lo + self.local_expert_num,
                                           w13_packed=e.w13_weight, w13_scale=e.w13_weight_scale, w2_packed=e.w2_weight,
                                           w2_scale=e.w2_weight_scale.float(), shared=shared, H=e.hidden_size,
                                           I=e.intermediate_size_per_partition, x_int8=x_int8,
                                           pertoken_scale=pertoken_scale,
                                           round_logits_bf16=self.gate.weight.dtype == torch.bfloat16,
                                           workspace=self._workspace, rows_dtype=self.rows_dtype, **routing)
            return out
        topk_weights, topk_ids = self._route(hidden_states, attn_metadata)
        x_in = hidden_states if x_int8 is None else x_int8
        return ops.moe_w8a8_layer(x_in, pertoken_scale, topk_weights, topk_ids, lo, lo + self.local_expert_num,
                                  e.w13_weight, e.w13_weight_scale, e.w2_weight, e.w2_weight_scale.float(), shared,
                                  H=e.hidden_size, I=e.intermediate_size_per_partition, workspace=self._workspace,
                                  rows_dtype=self.rows_dtype)
