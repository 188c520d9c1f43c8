"""CPU oracle for the expert-placement share of the MoE path (TEST INFRASTRUCTURE ONLY).

A plain-Python / numpy restatement of what the reference's placement planner contributes to a
forward step: the static tables built from a placement pattern and the two per-step operations.
Nothing in the shipped package imports this module; only tests do.

The table builder follows the reference's C++ step by step (one scan over the positions with the
``finish_table`` states and the growing candidate lists), on purpose: the library computes the same
tables from a closed form (first own copy, else same-host copies shared out by rank, else the others),
so a comparison of the two is a comparison of two formulations.

Pinning status (tests/test_placement.py):

* position_table / selector_table ... hand-written cases worked out on paper from the reference's
  rules; invariants on random patterns and on the placement patterns the reference's own tests hold
  (every selected position holds the expert asked for, an own copy always wins, a same-host copy wins
  over a distant one, the ranks of a host spread over the same-host copies); the closed form above,
  written independently in the test.
* remap_ids ......................... ``torch.nn.functional.embedding`` (the call the reference makes).
* record_activation ................. Python integers.
"""
from __future__ import annotations

import numpy as np


def position_table(pattern: np.ndarray, num_deploy: int) -> np.ndarray:
    """placement_mapping.cpp:223-257 (init_DeployedPositionToLogisticsIdMapping): for every layer, device
    ``r`` owns the positions [r*P, (r+1)*P), P = num_deploy // world; the experts it deploys fill them in
    ascending expert id; the rest stay -1."""
    world, layers, experts = pattern.shape
    per_device = num_deploy // world
    table = np.full((layers, num_deploy), -1, dtype=np.int32)
    for layer in range(layers):
        for rank in range(world):
            local = 0
            for expert in range(experts):
                if pattern[rank, layer, expert] == 1:
                    table[layer, per_device * rank + local] = expert
                    local += 1
    return table


def selector_table(pattern: np.ndarray, num_deploy: int, rank: int, devices_per_host: int) -> np.ndarray:
    """placement_mapping.cpp:374-427 (update_selector_layer), state for state: finish 2 = a copy on the rank
    itself was taken, 1 = a copy on the rank's host, 0 = only distant copies so far."""
    world, layers, experts = pattern.shape
    per_device = num_deploy // world
    positions = position_table(pattern, num_deploy)
    copies = pattern.astype(np.int64).sum(axis=0)            # [layers, experts]  (get_redundant_count)
    selector = np.zeros((layers, experts), dtype=np.int32)   # selector_host_ starts as zeros (:367)
    rank_host = rank // devices_per_host
    for layer in range(layers):
        finish = [0] * experts
        same_host = [[] for _ in range(experts)]
        distant = [[] for _ in range(experts)]
        for pos in range(num_deploy):
            e = int(positions[layer, pos])
            if e == -1:
                continue
            if copies[layer, e] == 1:
                selector[layer, e] = pos
                finish[e] = 1   # the reference stores `true`
                continue
            device = pos // per_device
            host = device // devices_per_host
            if finish[e] == 2:
                continue
            if device == rank:
                selector[layer, e] = pos
                finish[e] = 2
            elif finish[e] < 2 and host == rank_host:
                same_host[e].append(pos)
                selector[layer, e] = same_host[e][rank % len(same_host[e])]
                finish[e] = 1
            elif finish[e] < 1:
                distant[e].append(pos)
                selector[layer, e] = distant[e][rank % len(distant[e])]
    return selector


def remap_ids(ids: np.ndarray, expert_map: np.ndarray) -> np.ndarray:
    """omni_planner.py:273: ``embedding(token_expert_ids, expert_mapping).squeeze(-1)``: a table lookup."""
    return np.asarray(expert_map).reshape(-1)[np.asarray(ids)].astype(np.int32)


def record_activation(counts: np.ndarray, tokens_per_expert: np.ndarray, modulus: int) -> np.ndarray:
    """omni_planner.py:337-343: ``count = (count + expert_token_num) % max_activation_count`` (int64)."""
    return ((counts.astype(np.int64) + tokens_per_expert.astype(np.int64)) % np.int64(modulus)).astype(np.int64)
