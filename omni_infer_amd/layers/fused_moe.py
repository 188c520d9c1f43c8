"""Expert pipelines of the W8A8 MoE path on gfx950.

Mirror of omni/models/common/layers/moe/fused_moe/fused_moe.py for the functions that are on
the one-GPU path: ``fused_topk`` (:24-34), ``grouped_topk`` (:38-84),
``fused_experts_w8a8_allgather_ep`` (:489-538), ``gmm_expert`` (:541-575) and
``moe_expert_quant_farword`` (:663-687).  Same names, argument order and return values; the
``torch_npu`` operators underneath are replaced by the HIP operators of ``hip_ops``.
Weights are passed in the packed (frag16) layout that ``process_weights_after_loading`` makes.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import _lib as L
from .. import hip_ops as ops
from ..config import model_extra_config
from ..distributed import get_ep_group, get_world_group


def fused_topk(gating_output: torch.Tensor, topk: int, renormalize: bool):
    """fused_moe.py:24-34: softmax top-k, optional renormalisation by the plain sum."""
    T = gating_output.shape[0]
    w, ids = ops.moe_route(gating_output, None, topk, 1, 1, "softmax", L.OMNI_GROUP_MAX, False, False,
                           bool(renormalize), 1.0, 0.0)
    return w, ids, ops._row_idx(T, topk, gating_output.device)


def grouped_topk(hidden_states: torch.Tensor, gating_output: torch.Tensor, topk: int, renormalize: bool,
                 num_expert_group: int = 0, topk_group: int = 0, scoring_func: str = "softmax",
                 e_score_correction_bias: Optional[torch.Tensor] = None):
    """fused_moe.py:38-84: group score = max, masked experts score 0.0, weights are the
    (biased) scores, renormalise by the plain sum."""
    if scoring_func not in ("softmax", "sigmoid"):
        raise ValueError(f"Unsupported scoring function: {scoring_func}")
    T = gating_output.shape[0]
    w, ids = ops.moe_route(gating_output, e_score_correction_bias, topk, num_expert_group, topk_group, scoring_func,
                           L.OMNI_GROUP_MAX, True, True, bool(renormalize), 1.0, 0.0)
    return w, ids, ops._row_idx(T, topk, gating_output.device)


def fused_experts_w8a8_allgather_ep(hidden_states: torch.Tensor, pertoken_scale: torch.Tensor, w1: torch.Tensor,
                                    w2: torch.Tensor, w1_scale: torch.Tensor, w2_scale: torch.Tensor,
                                    topk_weights: torch.Tensor, topk_ids: torch.Tensor, n_routed_experts: int,
                                    is_prefill: bool, max_num_deployed_expert_per_rank: int,
                                    hidden_size: Optional[int] = None, intermediate_size: Optional[int] = None,
                                    rows_dtype: torch.dtype = torch.float32):
    """fused_moe.py:489-538.  hidden_states is int8 [T,H] with pertoken_scale [T]; topk_ids
    are global expert ids; only this GPU's experts are computed.  Returns bf16 [T,H], or None
    when the expert-parallel share is the whole model (the reference has no else branch,
    fused_moe.py:504).  ``rows_dtype`` (not in the reference): fp32 expert rows into the weighted
    sum, as the reference's fused GEMM2+finalize operator has them (:536), or bf16 rows."""
    redundancy = model_extra_config.parall_config.redundancy_shared_expert_num
    expert_parallel_size = get_ep_group().world_size - redundancy
    if expert_parallel_size <= 1:
        return None
    T, H = hidden_states.shape
    I = w1_scale.shape[-1] // 2
    lo = (get_world_group().rank_in_group - redundancy) * max_num_deployed_expert_per_rank
    hi = lo + n_routed_experts
    return ops.moe_w8a8_layer(hidden_states, pertoken_scale, topk_weights, topk_ids, lo, hi, w1, w1_scale, w2,
                              w2_scale.float(), None, H=H, I=I, rows_dtype=rows_dtype)


def fused_experts_w8a8_allgather_ep_a2(hidden_states: torch.Tensor, pertoken_scale: torch.Tensor, w1: torch.Tensor,
                                       w2: torch.Tensor, w1_scale: torch.Tensor, w2_scale: torch.Tensor,
                                       topk_weights: torch.Tensor, topk_ids: torch.Tensor, n_routed_experts: int,
                                       is_prefill: bool, max_num_deployed_expert_per_rank: int,
                                       smooth_scale: torch.Tensor, hidden_size: Optional[int] = None,
                                       intermediate_size: Optional[int] = None):
    """fused_moe.py:844-937, the A2 platform's form of the all-gather expert-parallel pipeline: ``smooth_scale``
    ([E_loc, I] fp32) multiplies the SwiGLU result before the row quantisation (``quant_scale`` of
    ``npu_dequant_swiglu_quant``, :907), and under ``pd_seperate_prefill`` the tail is a bf16 grouped GEMM followed
    by ``npu_moe_finalize_routing`` with bf16 routing weights (:909-918) instead of the fused GEMM2 + finalize
    (:919-927).  ``prefill_enable_long_seq`` (:873-875) trims the materialised sorted rows to the kept total; no
    sorted copy of the rows is made here (GEMM1 reads the tokens through the permutation), so there is nothing to
    trim.  The index patch-up of :879-884 only touches entries past the kept total, which nothing reads.
    Returns bf16 [T,H], or None when the expert-parallel share is the whole model (no else branch, :867)."""
    expert_parallel_size = get_ep_group().world_size
    if expert_parallel_size <= 1:
        return None
    opt = model_extra_config.operator_opt_config
    T, H = hidden_states.shape
    I = w1_scale.shape[-1] // 2
    lo = get_world_group().rank_in_group * max_num_deployed_expert_per_rank
    hi = lo + n_routed_experts
    if not opt.pd_seperate_prefill:
        return ops.moe_w8a8_layer(hidden_states, pertoken_scale, topk_weights, topk_ids, lo, hi, w1, w1_scale, w2,
                                  w2_scale.float(), None, H=H, I=I, quant_scale=smooth_scale)
    # row_idx_type 0 (:868): the sort's index is source -> slot, which is what the finalize step takes
    K = topk_ids.shape[1]
    p = ops.moe_permute(topk_ids, lo, hi, L.OMNI_IDX_TOKEN_MAJOR)
    M = T * K
    h_q, h_s, _ = ops.grouped_gemm1_swiglu_quant(hidden_states.contiguous(), pertoken_scale.reshape(-1).contiguous(),
                                                 p.sorted_src, L.OMNI_IDX_TOKEN_MAJOR, K, w1, w1_scale, p.offsets, H, I, M,
                                                 quant_scale=smooth_scale)
    rows, _ = ops.grouped_gemm2_dequant(h_q, h_s, w2, w2_scale.to(torch.bfloat16).float().contiguous(), p.offsets, H, I,
                                        out_dtype=torch.bfloat16)
    return ops.moe_combine(rows, topk_weights.to(torch.bfloat16), p.src_to_dst, L.OMNI_IDX_TOKEN_MAJOR, L.OMNI_ORDER_K)


def moe_expert_quant_farword(sorted_tokens: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, w1_scale: torch.Tensor,
                             w2_scale: torch.Tensor, expert_tokens: torch.Tensor, act_dtype, quant_mode,
                             dynamic_scale: Optional[torch.Tensor] = None):
    """fused_moe.py:663-687: rows already grouped by local expert (expert_tokens = counts).
    quant_mode 0: rows are bf16 and are quantised here; else rows are int8 with dynamic_scale."""
    if quant_mode:
        pertoken_scale = dynamic_scale
    else:
        sorted_tokens, pertoken_scale = ops.npu_dynamic_quant(sorted_tokens)
    M, H = sorted_tokens.shape
    I = w1_scale.shape[-1] // 2
    offsets = ops.group_offsets(expert_tokens)
    h_q, h_s, _ = ops.grouped_gemm1_swiglu_quant(sorted_tokens.contiguous(), pertoken_scale.reshape(-1).contiguous(),
                                                 None, 0, 1, w1, w1_scale, offsets, H, I, M)
    if not model_extra_config.operator_opt_config.opt_w2_scale_cast:
        w2_scale = w2_scale.to(torch.bfloat16)
    rows, _ = ops.grouped_gemm2_dequant(h_q, h_s, w2, w2_scale.float().contiguous(), offsets, H, I,
                                        out_dtype=torch.bfloat16 if act_dtype is None else act_dtype)
    return rows


def gmm_expert(x, expert_tokens, w1, w2, w1_scale, w2_scale, dynamic_scale=None, avg_tokens_per_expert=None):
    """fused_moe.py:541-575: same core with a bf16-rounded w2 scale (:569)."""
    hidden = x.size(-1)
    h = x.view(-1, hidden)
    M = h.shape[0]
    I = w1_scale.shape[-1] // 2
    offsets = ops.group_offsets(expert_tokens)
    h_q, h_s, _ = ops.grouped_gemm1_swiglu_quant(h.contiguous(), dynamic_scale.reshape(-1).contiguous(), None, 0, 1,
                                                 w1, w1_scale, offsets, hidden, I, M)
    rows, _ = ops.grouped_gemm2_dequant(h_q, h_s, w2, w2_scale.to(torch.bfloat16).float().contiguous(), offsets,
                                        hidden, I, out_dtype=torch.bfloat16)
    return rows
