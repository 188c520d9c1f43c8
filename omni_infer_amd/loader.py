"""Checkpoint -> parameters of one MoE block (compressed-tensors W8A8 safetensors).

Mirror of the part of ``DeepseekV3ForCausalLM.load_weights`` that fills a MoE block
(omni/models/deepseek/deepseek_v3.py:800-892): the stacked-parameter mapping for the shared
expert's ``gate_up_proj`` (:812-816), the expert mapping built by
``FusedMoE.make_expert_params_mapping`` (:818-822; vLLM's helper, bound at
omni/models/common/layers/moe/fused_moe/layer.py:174) and the fall-through to a parameter's own
``weight_loader`` (:876-889).  Checkpoint names look like

    model.layers.<L>.mlp.gate.weight                          fp32/bf16 [E, H]
    model.layers.<L>.mlp.gate.e_score_correction_bias         fp32 [E]
    model.layers.<L>.mlp.experts.<e>.gate_proj.weight         int8 [I, H]
    model.layers.<L>.mlp.experts.<e>.gate_proj.weight_scale   bf16 [I, 1]   (and weight_offset)
    model.layers.<L>.mlp.experts.<e>.{up_proj,down_proj}.*
    model.layers.<L>.mlp.shared_experts.{gate_proj,up_proj,down_proj}.{weight,weight_scale,weight_offset}

After loading, ``block.process_weights_after_loading()`` lays the int8 matrices out for the gfx950
kernels (the analogue of the reference's transpose + ``npu_format_cast``,
compressed_tensors_moe.py:94-114).  Nothing here touches the GPU unless the block's parameters
live there; files are read with ``safetensors.safe_open`` (no code from the file is executed).
"""
from __future__ import annotations

from typing import Iterable, Iterator, List, Sequence, Set, Tuple

import torch

STACKED_PARAMS_MAPPING = [
    # (param_name, shard_name, shard_id)          deepseek_v3.py:812-816
    ("gate_up_proj", "gate_proj", 0),
    ("gate_up_proj", "up_proj", 1),
]


def make_expert_params_mapping(ckpt_gate_proj_name: str, ckpt_down_proj_name: str, ckpt_up_proj_name: str,
                               num_experts: int) -> List[Tuple[str, str, int, str]]:
    """(param_name prefix, checkpoint name piece, expert_id, shard_id) for every expert and
    projection: gate -> w13 shard w1, up -> w13 shard w3, down -> w2 shard w2."""
    out = []
    for expert_id in range(num_experts):
        for shard_id, weight_name in (("w1", ckpt_gate_proj_name), ("w2", ckpt_down_proj_name),
                                      ("w3", ckpt_up_proj_name)):
            param = "experts.w13_" if weight_name in (ckpt_gate_proj_name, ckpt_up_proj_name) else "experts.w2_"
            out.append((param, f"experts.{expert_id}.{weight_name}.", expert_id, shard_id))
    return out


def iter_safetensors(paths: Sequence[str]) -> Iterator[Tuple[str, torch.Tensor]]:
    """(name, CPU tensor) for every tensor of every file, one tensor in memory at a time."""
    from safetensors import safe_open
    for path in paths:
        with safe_open(path, framework="pt", device="cpu") as f:
            for name in f.keys():
                yield name, f.get_tensor(name)


def default_weight_loader(param: torch.nn.Parameter, loaded_weight: torch.Tensor) -> None:
    if param.data.shape != loaded_weight.shape:
        raise RuntimeError(f"shape mismatch: parameter {tuple(param.data.shape)}, checkpoint {tuple(loaded_weight.shape)}")
    param.data.copy_(loaded_weight)


def load_moe_block(block: torch.nn.Module, weights: Iterable[Tuple[str, torch.Tensor]], prefix: str,
                   num_experts: int) -> Set[str]:
    """Fill ``block`` (a ``DeepseekMoE``) from ``weights``; names outside ``prefix`` are skipped.
    ``num_experts`` is the model's global expert count (experts of other ranks are dropped by
    ``FusedMoE.weight_loader``).  Returns the parameter names that received data."""
    if prefix and not prefix.endswith("."):
        prefix += "."
    expert_params_mapping = make_expert_params_mapping("gate_proj", "down_proj", "up_proj", num_experts)
    by_piece = {piece: (param_name, expert_id, shard_id) for param_name, piece, expert_id, shard_id in expert_params_mapping}
    params = dict(block.named_parameters())
    # a bias handed to the block as a plain attribute of the gate (deepseek_moe.py:154-157)
    loaded: Set[str] = set()
    for full_name, tensor in weights:
        if not full_name.startswith(prefix):
            continue
        name = full_name[len(prefix):]
        if "rotary_emb.inv_freq" in name:
            continue
        done = False
        for param_name, weight_name, shard_id in STACKED_PARAMS_MAPPING:
            if weight_name not in name:
                continue
            if "experts." in name and not name.startswith("shared_experts.") and name not in params:
                continue  # routed experts are handled by the expert mapping below
            mapped = name.replace(weight_name, param_name)
            if mapped.endswith(".bias") and mapped not in params:
                continue
            if mapped not in params:
                continue
            owner = _owner(block, mapped)
            owner.weight_loader(params[mapped], tensor, shard_id)
            loaded.add(mapped)
            done = True
            break
        if done:
            continue
        if name.startswith("experts."):
            # experts.<e>.<proj>.<leaf>
            parts = name.split(".")
            piece = ".".join(parts[:3]) + "."
            if piece in by_piece:
                param_name, expert_id, shard_id = by_piece[piece]
                mapped = name.replace(piece, param_name)
                if mapped in params:
                    block.experts.weight_loader(params[mapped], tensor, mapped, shard_id=shard_id, expert_id=expert_id)
                    loaded.add(mapped)
                continue
        if name.endswith(".bias") and name not in params:
            continue
        if name not in params:
            continue
        owner = _owner(block, name)
        loader = getattr(owner, "weight_loader", None)
        if loader is not None and not name.startswith("experts."):
            loader(params[name], tensor)
        else:
            default_weight_loader(params[name], tensor)
        loaded.add(name)
    return loaded


def _owner(block: torch.nn.Module, param_name: str) -> torch.nn.Module:
    mod = block
    for piece in param_name.split(".")[:-1]:
        mod = getattr(mod, piece)
    return mod
