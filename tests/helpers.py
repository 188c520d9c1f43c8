"""Shared builders for the parity tests: seeded inputs for the oracle and the device side."""
from __future__ import annotations

import torch

from oracle import moe_oracle as O


def gen(seed: int) -> torch.Generator:
    return torch.Generator().manual_seed(seed)


class Layer:
    """Seeded W8A8 expert weights in checkpoint layout plus the oracle's transposed views."""

    def __init__(self, n_local: int, H: int, I: int, seed: int = 0, shared: bool = False):
        g = gen(seed)
        self.n_local, self.H, self.I = n_local, H, I
        self.w13_ckpt, self.s13, self.w2_ckpt, self.s2 = O.make_expert_weights(n_local, H, I, g)
        self.w1_t = self.w13_ckpt.transpose(1, 2).contiguous()  # [E, H, 2I]  (oracle layout)
        self.w2_t = self.w2_ckpt.transpose(1, 2).contiguous()   # [E, I, H]
        self.shared = None
        if shared:
            a, sa, b, sb = O.make_expert_weights(1, H, I, g)
            self.sh13_ckpt, self.sh_s13, self.sh2_ckpt, self.sh_s2 = a[0], sa[0], b[0], sb[0]
            self.shared = (a[0].t().contiguous(), sa[0], b[0].t().contiguous(), sb[0])  # oracle layout

    def to_device(self, dev="cuda"):
        from omni_infer_amd import hip_ops as ops
        d = {}
        d["w13"] = ops.pack_weight(self.w13_ckpt.to(dev), 1)
        d["w2"] = ops.pack_weight(self.w2_ckpt.to(dev), 1)
        d["s13"] = self.s13.to(dev)
        d["s2"] = self.s2.to(dev)
        if self.shared is not None:
            d["sh13"] = ops.pack_weight(self.sh13_ckpt.to(dev), 1)
            d["sh2"] = ops.pack_weight(self.sh2_ckpt.to(dev), 1)
            d["sh_s13"] = self.sh_s13.to(dev)
            d["sh_s2"] = self.sh_s2.to(dev)
        return d


def tokens(T: int, H: int, seed: int, outlier_frac: float = 0.0) -> torch.Tensor:
    g = gen(seed)
    x = torch.randn(T, H, generator=g)
    if outlier_frac > 0:
        n = max(1, int(round(H * outlier_frac)))
        ch = torch.randperm(H, generator=g)[:n]
        x[:, ch] *= 50.0
    return x.to(torch.bfloat16)


def rel_err(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double().flatten(), b.double().flatten()
    return float((a - b).norm() / b.norm().clamp(min=1e-30))


def cosine(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double().flatten(), b.double().flatten()
    return float((a @ b) / (a.norm() * b.norm()).clamp(min=1e-30))
