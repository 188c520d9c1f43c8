"""One-GPU stand-in for the expert-parallel group the reference asks vLLM for.

The reference sizes the local expert share from ``get_ep_group().world_size`` and offsets it
by the rank (layer.py:206-209; compressed_tensors_moe.py:105-111; fused_moe.py:501-512).  This
build runs one GPU's share without any process group: the "group" is a plain record of which
share this GPU owns.  No collective is ever issued.
"""
from __future__ import annotations

from dataclasses import dataclass


@dataclass
class VirtualGroup:
    world_size: int = 1
    rank_in_group: int = 0


_EP = VirtualGroup()


def set_virtual_ep(world_size: int, rank: int = 0) -> None:
    """Declare that this GPU holds share ``rank`` of ``world_size`` equal expert shares."""
    if world_size < 1 or not (0 <= rank < world_size):
        raise ValueError("bad expert-parallel share")
    _EP.world_size, _EP.rank_in_group = world_size, rank


def get_ep_group() -> VirtualGroup:
    return _EP


def get_world_group() -> VirtualGroup:
    return _EP
