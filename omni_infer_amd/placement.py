"""Static expert placement on the MoE path: the part of the reference's placement planner that a forward
step touches.

Mirror of omni/accelerators/placement/omni_planner/expert_mapping.py (ExpertMapping) and
omni_planner.py (OmniPlanner) for a fixed placement pattern: the tables (which device deploys which
expert at which position, and the position a rank routes each logical expert to), the id remap of
``plan`` and the activation counters of ``record_activation``.  The tables are built by host code of the
library (omni_placement_tables), the two per-step operations are HIP kernels; nothing here has a CPU
fallback.  Dynamic re-placement (the optimiser threads, weight swapping over the collective library,
activation dumps to disk) is not built: ``enable_dynamic`` is always False here.
"""
from __future__ import annotations

import os
from typing import Optional, Tuple

import numpy as np
import torch
import yaml

from . import hip_ops as ops


def _read_config(config_file: Optional[str]) -> dict:
    """config.py:14-27: a YAML file; a missing file leaves every key at its default."""
    if not config_file:
        return {}
    try:
        with open(os.path.abspath(config_file), "r", encoding="utf-8") as fh:
            return yaml.safe_load(fh) or {}
    except FileNotFoundError:
        return {}


def _device(device) -> torch.device:
    """The reference's call sites say device="npu"; on this build that is the GPU."""
    if isinstance(device, str) and device.startswith("npu"):
        device = "cuda" + device[3:]
    return torch.device(device)


class ExpertMapping:
    """expert_mapping.py:12-281 for a static pattern.  ``pattern`` is [world, layers, experts] of 0/1 (an array,
    the path of a .npy file, or None for the base pattern: expert e on device e // (experts // world))."""

    def __init__(self, pattern=None, device="cuda", rank: int = 0, world_size: int = 1, num_devices_per_host: int = 8,
                 num_experts: int = 256, max_moe_layer_num: int = 58, max_redundant_per_rank: Optional[int] = None):
        self.device = _device(device)
        self.rank = rank
        self.world_size = world_size
        self.num_devices_per_host = num_devices_per_host
        self.max_moe_layer_num = max_moe_layer_num
        self.num_experts = num_experts
        self.max_redundant_per_rank = max_redundant_per_rank
        self.placement_pattern_cpu = self._load_placement_pattern_with_validation(pattern)
        self.placement_pattern = self.placement_pattern_cpu
        world = self.placement_pattern_cpu.shape[0]
        # expert_mapping.py:33, :43: every device gets the same number of positions, the largest layer's share
        self.max_num_deployed_expert_per_rank = max(max(self.get_deployed_experts_per_layer()) // world, 1)
        num_deploy = self.max_num_deployed_expert_per_rank * world
        pos, sel = ops.placement_tables(self.placement_pattern_cpu, rank, num_devices_per_host, num_deploy)
        self.position_to_expert = pos                       # CPU [layers, num_deploy]
        self.selector_cpu = sel                             # CPU [layers, experts]
        # expert_mapping.py:39: [layers, experts, 1] int32 on the device; plan() looks ids up in one layer's slice
        self.selector = sel.to(self.device).unsqueeze(-1)
        self.local_expert_offsets = self._calc_expert_offset_each_layer()

    def _load_placement_pattern_with_validation(self, pattern) -> torch.Tensor:
        """expert_mapping.py:57-97."""
        if pattern is None:
            per = self.num_experts // self.world_size
            arr = np.zeros((self.world_size, self.max_moe_layer_num, self.num_experts), dtype=np.int32)
            for r in range(self.world_size):
                arr[r, :, r * per:(r + 1) * per] = 1
        elif isinstance(pattern, (str, os.PathLike)):
            if not os.path.exists(pattern):
                raise FileNotFoundError(f"[Placement-Error]: Placement pattern file not found: {pattern}")
            arr = np.load(pattern, allow_pickle=False).astype(np.int32)
        else:
            arr = np.asarray(pattern.cpu() if isinstance(pattern, torch.Tensor) else pattern).astype(np.int32)
        want = (self.world_size, self.max_moe_layer_num, self.num_experts)
        if arr.shape != want:
            raise ValueError(f"[Placement-Error]: pattern.shape[{arr.shape}] is not equals to (world_size[{want[0]}], "
                             f"layers[{want[1]}], num_experts[{want[2]}])")
        return torch.from_numpy(np.ascontiguousarray(arr))

    def get_selector(self) -> torch.Tensor:
        return self.selector

    def is_moe_layer(self, layer_idx_moe: int) -> bool:
        return layer_idx_moe < self.max_moe_layer_num

    def is_expert_on_current_rank(self, layer_idx_moe: int, expert_id: int, current_rank: int,
                                  experts_per_rank: int) -> Tuple[bool, int]:
        """expert_mapping.py:101-126: (deployed on that rank, number of deployed experts with a lower id there)."""
        if not self.is_moe_layer(layer_idx_moe):
            return self._default_deployment_check(expert_id, current_rank, experts_per_rank)
        row = self.placement_pattern_cpu[current_rank, layer_idx_moe]
        return bool(row[expert_id] > 0), int(row[:expert_id].sum().item())

    @staticmethod
    def _default_deployment_check(expert_id: int, current_rank: int, experts_per_rank: int) -> Tuple[bool, int]:
        """expert_mapping.py:128-139."""
        start = current_rank * experts_per_rank
        inside = start <= expert_id < start + experts_per_rank
        return inside, (expert_id - start if inside else -1)

    def get_num_of_redundant_experts(self, moe_layer_idx: int, num_expert_per_device_origin: int = 16,
                                     rank_device: int = 0) -> int:
        """expert_mapping.py:141-164."""
        if self.max_redundant_per_rank is not None:
            return self.max_redundant_per_rank
        here = self.placement_pattern_cpu[rank_device][moe_layer_idx]
        return round(here.sum().item() - num_expert_per_device_origin)

    def get_world_size(self) -> int:
        return self.placement_pattern_cpu.shape[0]

    def get_total_num_expert(self) -> int:
        return self.placement_pattern_cpu.shape[2]

    def get_total_num_layers(self) -> int:
        return self.placement_pattern_cpu.shape[1]

    def get_deployed_experts_per_layer(self) -> list:
        """expert_mapping.py:178-185."""
        if self.max_redundant_per_rank is not None:
            return [self.get_total_num_expert() + self.max_redundant_per_rank * self.get_world_size()] * self.get_total_num_layers()
        return self.placement_pattern_cpu.sum(dim=(0, 2)).tolist()

    def get_redundant_enable_per_layer(self) -> list:
        """expert_mapping.py:187-197."""
        if self.max_redundant_per_rank is not None:
            return [self.max_redundant_per_rank != 0] * self.get_total_num_layers()
        return [v != self.get_total_num_expert() for v in self.get_deployed_experts_per_layer()]

    def _calc_expert_offset_each_layer(self) -> torch.Tensor:
        """expert_mapping.py:199-214: experts deployed on the ranks before each rank, per layer."""
        counts = self.placement_pattern_cpu.sum(dim=-1)
        offsets = torch.zeros_like(counts)
        offsets[1:] = torch.cumsum(counts, dim=0)[:-1]
        return offsets

    def get_local_expert_indices_offset(self, layer_idx_moe: int, current_rank: int, default_experts_per_rank: int = 0) -> int:
        """expert_mapping.py:216-220."""
        if self.max_redundant_per_rank is not None:
            return self.rank * self.max_num_deployed_expert_per_rank
        return int(self.local_expert_offsets[current_rank, layer_idx_moe].item())

    def get_max_num_deployed_expert_per_rank(self) -> int:
        return self.max_num_deployed_expert_per_rank


class OmniPlanner:
    """omni_planner.py:44-343 for a static placement.  Takes the reference's constructor arguments; the pattern and
    ``max_moe_layer_num`` come from the YAML ``config_file`` (keys ``pattern_path``, ``max_moe_layer_num``,
    ``enable_dump``) or, in place of a file, from the keyword arguments of the same names."""

    def __init__(self, config_file: Optional[str] = None, device: str = "cuda", rank: int = 0, world_size: int = 1,
                 num_devices_per_host: int = 16, num_experts: int = 256, num_redundancy_shared_expert_rank: int = 0,
                 pattern=None, max_moe_layer_num: Optional[int] = None, enable_dump: bool = False):
        cfg = _read_config(config_file)
        self.max_moe_layer_num = cfg.get("max_moe_layer_num", max_moe_layer_num)
        if self.max_moe_layer_num is None:
            raise ValueError("[Placement-Error]-max_moe_layer_num is not defined")
        self.device = _device(device)
        # omni_planner.py:127-155: ranks that only hold redundant shared experts are not part of the expert pattern
        self.rank = rank - num_redundancy_shared_expert_rank
        self.world_size = world_size - num_redundancy_shared_expert_rank
        self.num_devices_per_host = num_devices_per_host
        self.enable_dynamic = False
        self.enable_dump = bool(cfg.get("enable_dump", enable_dump))
        if pattern is None and cfg.get("pattern_path"):
            pattern = cfg["pattern_path"]
            if config_file and not os.path.isabs(pattern):
                pattern = os.path.join(os.path.dirname(os.path.abspath(config_file)), pattern)
        self.expert_mapping = ExpertMapping(pattern, self.device, self.rank, self.world_size, num_devices_per_host,
                                            num_experts, self.max_moe_layer_num)
        # omni_planner.py:161-166
        self.npu_activation_count = torch.zeros((self.expert_mapping.get_total_num_layers(),
                                                 self.get_max_num_deployed_expert_per_rank()),
                                                device=self.device, dtype=torch.int64)
        self.max_activation_count = int(1e16)
        self.selector = self.expert_mapping.get_selector()
        self.redundant_enable_per_layer = self.expert_mapping.get_redundant_enable_per_layer()

    def is_moe_layer(self, layer_idx_moe: int) -> bool:
        return layer_idx_moe < self.max_moe_layer_num

    def get_max_num_deployed_expert_per_rank(self) -> int:
        return self.expert_mapping.get_max_num_deployed_expert_per_rank()

    def is_expert_on_current_rank(self, layer_id: int, expert_id: int, current_rank: int, experts_per_rank: int):
        return self.expert_mapping.is_expert_on_current_rank(layer_id, expert_id, current_rank, experts_per_rank)

    def expert_mapping_on_current_layer(self, layer_idx_moe: int, is_prefill: bool = False) -> Optional[torch.Tensor]:
        """omni_planner.py:220-226: the layer's slice [experts, 1] of the selector."""
        if not self.is_moe_layer(layer_idx_moe):
            return None
        return self.selector[layer_idx_moe]

    def plan(self, layer_idx_moe: Optional[int] = None, tokens: Optional[torch.Tensor] = None,
             token_expert_ids: Optional[torch.Tensor] = None, token_expert_scores: Optional[torch.Tensor] = None,
             top_k: int = 8, expert_mapping: Optional[torch.Tensor] = None, is_prefill: bool = True):
        """omni_planner.py:244-274: ids -> deployed positions, by the table of the layer."""
        if not self.is_moe_layer(layer_idx_moe):
            return tokens, token_expert_ids, token_expert_scores
        if expert_mapping is None:
            expert_mapping = self.selector[layer_idx_moe]
        return tokens, ops.remap_ids(token_expert_ids, expert_mapping), token_expert_scores

    @staticmethod
    def get_deepseek_v3_moe_layer_idx(prefix: str, first_k_dense_replace: int = 3) -> int:
        """omni_planner.py:277-306: ``model.layers.{N}.mlp.experts`` -> N - first_k_dense_replace."""
        return int(prefix.split(sep=".")[2]) - first_k_dense_replace

    def get_num_of_redundant_experts(self, moe_layer_idx: int, num_expert_per_device_origin: int = 16,
                                     rank_device: int = 0) -> int:
        if not self.is_moe_layer(moe_layer_idx):
            return 0
        return self.expert_mapping.get_num_of_redundant_experts(moe_layer_idx, num_expert_per_device_origin, rank_device)

    def record_activation(self, layer_idx_moe: int, expert_token_num: torch.Tensor, is_prefill: bool = True) -> None:
        """omni_planner.py:337-343 (the reference moves the decode update to a side stream; here it is one small
        launch on the current stream)."""
        if self.is_moe_layer(layer_idx_moe):
            ops.record_activation(self.npu_activation_count[layer_idx_moe], expert_token_num, self.max_activation_count)
