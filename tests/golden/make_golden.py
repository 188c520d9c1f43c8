"""Writes the golden fixtures of the toy configuration from the CPU oracle.

The reference ships no golden vector for the MoE path (its arithmetic lives in closed torch_npu
kernels and none of its tests touches them), so the fixtures freeze this repository's oracle:
BASELINE config 1 (8 experts, H=1024, I=512, top-2 softmax renormalised, 64 tokens, seed 0),
inputs by seed, outputs of every stage of both pipelines.  Run: python -m tests.golden.make_golden
"""
from __future__ import annotations

import os

import torch

from oracle import moe_oracle as O


def toy_config1():
    g = torch.Generator().manual_seed(0)
    E, H, I, K, T = 8, 1024, 512, 2, 64
    w13, s13, w2, s2 = O.make_expert_weights(E, H, I, g)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    gate = (torch.randn(E, H, generator=g) * 0.02).to(torch.bfloat16)
    logits = x.float() @ gate.float().t()
    w, ids, row_idx = O.route_softmax_topk(logits, K, True)
    xq, xs = O.dynamic_quant(x)
    w1_t, w2_t = w13.transpose(1, 2).contiguous(), w2.transpose(1, 2).contiguous()
    out_f, st = O.fused_experts_w8a8_allgather_ep(xq, xs, w1_t, w2_t, s13, s2, w, ids, (0, E), return_stages=True)
    out_u = O.fused_experts_w8a8(x, w1_t, w2_t, s13, s2, w, ids, row_idx)

    def digest(t):  # a checksum in place of the full int32 accumulator matrices
        return torch.tensor([int(t.long().sum()), int((t.long() * t.long()).sum() % (1 << 61))])
    return {
        "logits": logits, "topk_w": w, "topk_ids": ids, "x_q_sum": digest(xq), "x_s": xs,
        "expanded_x_idx": st["idx"], "counts": st["counts"], "acc1_digest": digest(st["acc1"]),
        "h_q_digest": digest(st["h_q"]), "h_s": st["h_s"], "acc2_digest": digest(st["acc2"]),
        "out_fused": out_f, "out_unfused": out_u,
    }


if __name__ == "__main__":
    here = os.path.dirname(os.path.abspath(__file__))
    torch.save(toy_config1(), os.path.join(here, "toy_config1.pt"))
    print("wrote", os.path.join(here, "toy_config1.pt"))
