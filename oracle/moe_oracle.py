"""CPU oracle for the W8A8 dynamic-quant fused-MoE path (TEST INFRASTRUCTURE ONLY).

This module is a PyTorch-CPU-eager restatement of the operator semantics that
omni-infer's MoE hot path asks of ``torch_npu`` (whose source is a third-party,
un-vendored dependency: torch_npu 2.5.1 on CANN 8.1.RC1, see
tests/README.md:10-18 of the reference).  It is the checker that the HIP kernels
are compared against.  Nothing in the shipped package imports it; only tests,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do.

Every function cites the reference call site whose semantics it restates
(paths relative to the reference tree).

Arithmetic that the reference leaves to closed kernels is fixed here so that a
device implementation can match it bit for bit:

* all floating point is IEEE fp32, one rounding per written operation
  (no fused multiply-add), divisions are true divisions;
* ``exp`` is the routine ``exp_spec`` below (Cody-Waite reduction plus the
  Cephes ``expf`` polynomial, evaluated by Horner with separate multiplies
  and adds); sigmoid and SiLU are built from it with one division;
* reductions whose order matters have a stated order: the softmax
  denominator is summed lane-wise (``V`` consecutive experts per lane,
  ascending, V = ceil(E/64) rounded up to a power of two) and then by a 64-lane butterfly (masks 1,2,4,8,16,32);
  top-k renormalisation sums in output order; the weighted combine adds rows
  in ascending sorted-slot order (fused GEMM2+finalize) or ascending ``k``
  (``npu_moe_finalize_routing``);
* ties in any top-k go to the lower index; outputs are in descending score.

Pinning status (what independent evidence each function is checked against in
tests/test_oracle_pins.py):

* exp_spec / sigmoid_spec / silu_spec ... torch.exp / sigmoid / F.silu within
  4 ulp over a dense sweep; monotonicity; exact values at 0.
* fma32 / gate_logits_spec ... exact rational arithmetic (fractions) on random
  and constructed half-way cases; fp64 matmul (a dropped term, a transposed
  operand or a wrong slice boundary fails); invariance under the split of the
  slices over wavefronts is a property of the device test.
* route_noaux_tc ........ transformers DeepseekV3TopkRouter arithmetic
  (library routine, ids as sets + weights), brute force over all subsets on
  tiny E, invariants (distinct ids, group membership, sum of weights).
* route_grouped_topk .... line-by-line torch restatement of the reference's
  own pure-torch function (fused_moe.py:38-84), run side by side.
* route_softmax_topk .... torch.softmax + torch.topk.
* dynamic_quant ......... closed-form invariants (|q|max = 127, |x - q s| <=
  s/2, idempotence), numpy float64 recomputation.
* moe_init_routing_v1/v2  permutation invariants, bincount, numpy stable
  argsort.
* grouped_matmul_int32 .. fp64 matmul witness, per-expert loop.
* dequant_swiglu_quant, grouped_matmul_dequant, quant_matmul, swiglu_bf16,
  finalize ... closed forms in float64 from the exact integer products (a
  wrong group's scale, a missing per-token scale, swapped halves must fail),
  and the end-to-end dense brute force (every token through every selected
  expert without any permutation).
* fused_experts_w8a8_allgather_ep_a2 ... permutation-free fp64 brute force with the
  smoothing factors inside (dropping them, or applying them after the row
  quantisation instead of before, fails); with factors of one the bits of
  fused_experts_w8a8_allgather_ep; the bf16 tail against the same brute force
  within the bf16 bar, and != the fp32-row tail.
* moe_expert_quant_forward ... permutation-free fp64 witness; its second
  stage within one bf16 step of the fp64 closed form with the w2 scale it was
  asked to use (a skipped bf16 rounding of that scale fails).
* deepseek_moe_forward ... fp64 witness of the whole block built from the
  transformers router, the dense brute force and an fp64 shared expert (a
  wrong expert range or a missing shared expert fails); the rounding points
  of the final add (bf16 + bf16) by composition with the block without a
  shared expert.
* add_rms_norm / add_rms_norm_dynamic_quant (the producer in front of the
  block) ... torch.nn.functional.rms_norm in float64 (library routine) within
  one bf16 step, closed forms on constant and zero rows, power-of-two scale
  invariance, unit RMS, the quantisation invariants; its square root against
  numpy's (tests/test_norm.py).

Parity unpinned by the reference itself: the reference holds no test, golden
vector or fixture for this path, and the rounding mode, zero-row behaviour,
tie-breaking, intra-expert order, multiplication order and exp implementation
of the closed kernels cannot be observed here.  They are fixed by the
definitions above.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

F32 = torch.float32


def _c(v: float) -> torch.Tensor:
    return torch.tensor(v, dtype=F32)


# --------------------------------------------------------------------------
# Specified transcendental: exp, sigmoid, SiLU
# --------------------------------------------------------------------------
EXP_LO = -87.0
EXP_HI = 87.0
LOG2E = 1.44269504088896341
LN2_HI = 0.693359375
LN2_LO = -2.12194440e-4
EXP_P = (1.9875691500e-4, 1.3981999507e-3, 8.3334519073e-3,
         4.1665795894e-2, 1.6666665459e-1, 5.0000001201e-1)


def exp_spec(x: torch.Tensor) -> torch.Tensor:
    """fp32 exp with a fixed operation sequence (one rounding per operation).

    x is clamped to [-87, 87]; t = x*log2(e); n = rint(t); r = (x - n*LN2_HI)
    - n*LN2_LO; p = Horner(EXP_P, r); y = (p*(r*r) + r) + 1; result = y * 2^n.
    """
    x = x.to(F32)
    x = torch.clamp(x, min=EXP_LO, max=EXP_HI)
    n = torch.round(x * _c(LOG2E))
    r = x - n * _c(LN2_HI)
    r = r - n * _c(LN2_LO)
    p = torch.full_like(r, EXP_P[0])
    for coef in EXP_P[1:]:
        p = p * r
        p = p + _c(coef)
    y = p * (r * r)
    y = y + r
    y = y + _c(1.0)
    two_n = ((n.to(torch.int32) + 127) << 23).view(F32)
    return y * two_n


def sigmoid_spec(x: torch.Tensor) -> torch.Tensor:
    """1 / (1 + exp_spec(-x))."""
    x = x.to(F32)
    return _c(1.0) / (_c(1.0) + exp_spec(-x))


def silu_spec(x: torch.Tensor) -> torch.Tensor:
    """x / (1 + exp_spec(-x))."""
    x = x.to(F32)
    return x / (_c(1.0) + exp_spec(-x))


# --------------------------------------------------------------------------
# Gate projection with a stated summation order
# --------------------------------------------------------------------------
GATE_SLICE = 128   # reduction elements of one fused-multiply-add chain
GATE_GROUP = 8     # slices added up before the groups are


def fma32(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor) -> torch.Tensor:
    """fp32 fused multiply-add, a*b + c with a single rounding (round to nearest even), for fp32
    tensors without overflow or subnormal results.

    The product of two fp32 numbers is exact in fp64 (48 significant bits).  The fp64 sum p + c is
    rounded once to 53 bits; rounding that again to 24 bits differs from the single rounding only when
    the fp64 sum lies exactly half way between two neighbouring fp32 numbers while the exact sum does
    not.  The exact error of the fp64 addition (two-sum) tells on which side the exact sum lies."""
    p = a.to(torch.float64) * b.to(torch.float64)
    cd = c.to(torch.float64)
    s = p + cd
    r = s.to(F32)
    bb = s - p
    err = (p - (s - bb)) + (cd - bb)                       # exact: s + err == p + c
    rd = r.to(torch.float64)
    toward = torch.where(s > rd, torch.full_like(r, float("inf")), torch.full_like(r, float("-inf")))
    other = torch.nextafter(r, toward)
    tie = (rd != s) & ((rd - s).abs() == (other.to(torch.float64) - s).abs())
    fix = tie & (err != 0)
    if bool(fix.any()):
        hi = torch.maximum(r, other)
        lo = torch.minimum(r, other)
        r = torch.where(fix, torch.where(err > 0, hi, lo), r)
    return r


def gate_logits_spec(x: torch.Tensor, w: torch.Tensor, round_bf16: bool = False) -> torch.Tensor:
    """``router_logits, _ = self.gate.forward(hidden_states.float())`` (omni/models/common/layers/moe/
    deepseek_moe.py:147-152,253,329): logits[t,e] = sum_k x[t,k] * w[e,k] in fp32, here with the stated
    order of the device library (the reference leaves the order to its BLAS):

    the reduction is cut into slices of 128 elements; a slice is a chain of fused multiply-adds over
    ascending k starting from +0; 8 consecutive slices are added left to right into a group sum; the
    group sums are added left to right.  ``round_bf16``: the bf16 gate of deepseek_v3_a2.py:607-613
    hands bf16 logits to the router.  x [T,H] (bf16 or fp32), w [E,H] (fp32 or bf16), H % 128 == 0."""
    xf, wf = x.to(F32), w.to(F32)
    T, H = xf.shape
    E = wf.shape[0]
    assert H % GATE_SLICE == 0
    n_slices = H // GATE_SLICE
    wt = wf.t().contiguous()                                # [H, E]
    total = None
    for g0 in range(0, n_slices, GATE_GROUP):
        q = None
        for s_ in range(g0, min(g0 + GATE_GROUP, n_slices)):
            acc = torch.zeros(T, E, dtype=F32)
            for k in range(s_ * GATE_SLICE, (s_ + 1) * GATE_SLICE):
                acc = fma32(xf[:, k:k + 1], wt[k:k + 1, :], acc)
            q = acc if q is None else q + acc
        total = q if total is None else total + q
    if round_bf16:
        total = total.to(torch.bfloat16).to(F32)
    return total


# --------------------------------------------------------------------------
# Routing (C1, C2, C3)
# --------------------------------------------------------------------------
def _topk_desc_low_index(scores: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Top-k along the last dim: descending value, ties to the lower index."""
    order = torch.sort(scores, dim=-1, descending=True, stable=True).indices[..., :k]
    return torch.gather(scores, -1, order), order


def _seq_sum(w: torch.Tensor) -> torch.Tensor:
    """Sum over the last dim in ascending index order, fp32, one add at a time."""
    acc = w[..., 0].clone()
    for j in range(1, w.shape[-1]):
        acc = acc + w[..., j]
    return acc


def route_noaux_tc(logits: torch.Tensor, bias: torch.Tensor, top_k: int, n_group: int,
                   topk_group: int, routed_scaling_factor: float, eps: float = 1e-20
                   ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Sigmoid + correction-bias group-limited top-k ("noaux_tc").

    Restates ``torch_npu.npu_moe_gating_top_k(logits.float(), k, bias, k_group,
    group_count, group_select_mode=1, renorm=0, norm_type=1,
    routed_scaling_factor, eps)`` as called at
    omni/models/common/layers/moe/fused_moe/layer.py:341-351.

    s = sigmoid(logits); c = s + bias; a group's score is the sum of its two
    largest c; the ``topk_group`` best groups are kept (ties: lower group id);
    the ``top_k`` largest c among kept groups are selected (ties: lower id,
    output in descending c); w = s[ids] / (sum_k s[ids] + eps) * scale.
    Returns (weights fp32 [T,K], ids int32 [T,K]).
    """
    logits = logits.to(F32)
    T, E = logits.shape
    s = sigmoid_spec(logits)
    c = s + bias.to(F32).unsqueeze(0)
    gs = c.view(T, n_group, E // n_group)
    top2, _ = _topk_desc_low_index(gs, 2)
    group_scores = top2[..., 0] + top2[..., 1]
    _, gidx = _topk_desc_low_index(group_scores, topk_group)
    gmask = torch.zeros(T, n_group, dtype=torch.bool)
    gmask.scatter_(1, gidx, True)
    emask = gmask.unsqueeze(-1).expand(T, n_group, E // n_group).reshape(T, E)
    masked = torch.where(emask, c, torch.full_like(c, float("-inf")))
    _, ids = _topk_desc_low_index(masked, top_k)
    w = torch.gather(s, 1, ids)
    denom = _seq_sum(w) + _c(eps)
    w = w / denom.unsqueeze(-1)
    w = w * _c(routed_scaling_factor)
    return w, ids.to(torch.int32)


def route_grouped_topk(logits: torch.Tensor, top_k: int, renormalize: bool, n_group: int,
                       topk_group: int, scoring_func: str = "softmax",
                       bias: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """The reference's pure-torch ``grouped_topk``
    (omni/models/common/layers/moe/fused_moe/fused_moe.py:38-84).

    Scores by softmax or sigmoid (+ optional bias); group score = max; experts
    outside the kept groups get score 0.0 (not -inf, fused_moe.py:69); weights
    are the (biased) masked scores; renormalise by the plain sum
    (fused_moe.py:75-76); ``row_idx[n,k] = k*T + n`` (fused_moe.py:80-81).
    The caller multiplies by routed_scaling_factor (layer.py:339).
    The reference asks torch.topk for ``sorted=False``; here the order is
    fixed: descending, ties to the lower index.
    """
    logits = logits.to(F32)
    T, E = logits.shape
    if scoring_func == "softmax":
        scores = softmax_spec(logits)
    elif scoring_func == "sigmoid":
        scores = sigmoid_spec(logits)
    else:
        raise ValueError(f"Unsupported scoring function: {scoring_func}")
    if bias is not None:
        scores = scores + bias.to(F32).unsqueeze(0)
    group_scores = scores.view(T, n_group, -1).max(dim=-1).values
    _, gidx = _topk_desc_low_index(group_scores, topk_group)
    gmask = torch.zeros(T, n_group, dtype=torch.bool)
    gmask.scatter_(1, gidx, True)
    emask = gmask.unsqueeze(-1).expand(T, n_group, E // n_group).reshape(T, E)
    tmp = torch.where(emask, scores, torch.zeros_like(scores))
    w, ids = _topk_desc_low_index(tmp, top_k)
    if renormalize:
        w = w / _seq_sum(w).unsqueeze(-1)
    ids = ids.to(torch.int32)
    row_idx = torch.arange(T * top_k, dtype=torch.int32).reshape(top_k, T).transpose(1, 0).contiguous()
    return w, ids, row_idx


def _butterfly_sum64(v: torch.Tensor) -> torch.Tensor:
    """All-reduce sum over a last dim of 64 by xor butterfly, masks 1..32."""
    lane = torch.arange(64)
    for mask in (1, 2, 4, 8, 16, 32):
        v = v + v[..., lane ^ mask]
    return v[..., 0]


def softmax_spec(logits: torch.Tensor) -> torch.Tensor:
    """fp32 softmax over the last dim with a fixed summation order.

    e = exp_spec(x - max); lane l owns the V consecutive entries [V*l, V*l+V)
    (V = ceil(E/64) rounded up to a power of two; missing entries count as 0)
    and adds them in ascending order; the 64 lane sums are combined by the butterfly above; p = e / sum.
    """
    logits = logits.to(F32)
    T, E = logits.shape
    V = 1
    while 64 * V < E:
        V *= 2
    m = logits.max(dim=-1, keepdim=True).values
    e = exp_spec(logits - m)
    pad = torch.zeros(T, 64 * V, dtype=F32)
    pad[:, :E] = e
    lanes = _seq_sum(pad.view(T, 64, V)) if V > 1 else pad.view(T, 64)
    tot = _butterfly_sum64(lanes)
    return e / tot.unsqueeze(-1)


def route_softmax_topk(logits: torch.Tensor, top_k: int, renormalize: bool
                       ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``fused_topk`` = ``npu_moe_gating_top_k_softmax`` + optional renormalise
    (omni/models/common/layers/moe/fused_moe/fused_moe.py:24-34).
    Returns (weights, ids int32, row_idx) with row_idx[n,k] = k*T + n.
    """
    T = logits.shape[0]
    p = softmax_spec(logits)
    w, ids = _topk_desc_low_index(p, top_k)
    if renormalize:
        w = w / _seq_sum(w).unsqueeze(-1)
    row_idx = torch.arange(T * top_k, dtype=torch.int32).reshape(top_k, T).transpose(1, 0).contiguous()
    return w, ids.to(torch.int32), row_idx


# --------------------------------------------------------------------------
# Per-token dynamic quantisation (C4)
# --------------------------------------------------------------------------
def dynamic_quant(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """``torch_npu.npu_dynamic_quant(x)`` (omni/models/common/layers/moe/
    deepseek_moe.py:247,323; compressed_tensors_moe.py:241,247).

    Per row: s = max|x| / 127 in fp32; q = clamp(rint(x / s), -128, 127) with a
    true division and round-half-even.  An all-zero row gives s = 0, q = 0.
    """
    xf = x.to(F32)
    amax = xf.abs().amax(dim=-1)
    s = amax / _c(127.0)
    safe = torch.where(s > 0, s, torch.ones_like(s))
    q = torch.round(xf / safe.unsqueeze(-1))
    q = torch.where((s > 0).unsqueeze(-1), q, torch.zeros_like(q))
    q = torch.clamp(q, -128, 127).to(torch.int8)
    return q, s


# --------------------------------------------------------------------------
# Residual add + RMSNorm (+ dynamic quant): the producer in front of the block
# --------------------------------------------------------------------------
def _sqrt_rn(v: torch.Tensor) -> torch.Tensor:
    """Correctly rounded fp32 square root.  torch's vectorised fp32 sqrt on x86 is off by one unit in
    the last place for about 0.7 % of inputs (checked against numpy and against the rounded fp64 root);
    the fp64 root rounded to fp32 is the correctly rounded result (53 >= 2*24 + 2 bits)."""
    return torch.sqrt(v.to(torch.float64)).to(F32)


def add_rms_norm(x: torch.Tensor, residual: Optional[torch.Tensor], weight: torch.Tensor, eps: float
                 ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """``RMSNorm.forward`` (omni/models/common/layers/layernorm.py:13-32):
    ``npu_add_rms_norm(x, residual, weight, eps)`` -> (y, residual_out), or
    ``npu_rms_norm(x, weight, eps)`` when there is no residual.

    s = float(x) + float(residual); residual_out = s rounded to the input dtype;
    y = ((s * r) * float(weight)) rounded to the input dtype, r = 1 / sqrt(mean(s*s) + eps) with a
    correctly rounded root and a true division.
    The mean's sum has a fixed order: the row is cut into vectors of 8 elements; slot t of 256
    owns vectors t, t+256, ... and adds their squares in index order; the 64 slots of each of the
    four groups are combined by the xor butterfly (1..32) and the groups as ((g0+g1)+g2)+g3.
    """
    dt = x.dtype
    T, H = x.shape
    assert H % 8 == 0
    s = x.to(F32)
    res_out = None
    if residual is not None:
        s = s + residual.to(F32)
        res_out = s.to(dt)
    nvec = H // 8
    rounds = (nvec + 255) // 256
    sq = torch.zeros(T, rounds * 256 * 8, dtype=F32)
    sq[:, :H] = s * s
    sq = sq.view(T, rounds, 256, 8)
    acc = torch.zeros(T, 256, dtype=F32)
    for i in range(rounds):
        for j in range(8):
            acc = acc + sq[:, i, :, j]      # absent vectors add exact zeros
    groups = [_butterfly_sum64(acc[:, 64 * g:64 * g + 64].contiguous()) for g in range(4)]
    total = ((groups[0] + groups[1]) + groups[2]) + groups[3]
    mean = total / _c(float(H))
    r = _c(1.0) / _sqrt_rn(mean + _c(eps))
    y = ((s * r.unsqueeze(-1)) * weight.to(F32)).to(dt)
    return y, res_out


def add_rms_norm_dynamic_quant(x: torch.Tensor, residual: Optional[torch.Tensor], weight: torch.Tensor, eps: float):
    """``RMSNorm.forward(..., quant_symbol=True)`` (layernorm.py:21-25): the normalised
    tensor, in the model dtype, goes through ``npu_dynamic_quant``.
    Returns (x_int8, pertoken_scale, residual_out)."""
    y, res_out = add_rms_norm(x, residual, weight, eps)
    q, sc = dynamic_quant(y)
    return q, sc, res_out


# --------------------------------------------------------------------------
# Permutation (C5)
# --------------------------------------------------------------------------
def moe_init_routing_v2(x: torch.Tensor, topk_ids: torch.Tensor, scale: Optional[torch.Tensor],
                        expert_range: Tuple[int, int]):
    """``npu_moe_init_routing_v2(..., active_expert_range=[lo,hi), row_idx_type=1,
    expert_tokens_num_type=1, quant_mode=-1, drop_pad_mode=0)``
    (omni/models/common/layers/moe/fused_moe/fused_moe.py:514-515).

    Stable sort of the flattened (n*K + k) assignments by expert id, keeping
    those with lo <= id < hi.  Returns (rows [M,H], expanded_x_idx int32 [M]
    = flat source index of each sorted slot, counts int64 [hi-lo], gathered
    scale fp32 [M] or None).
    """
    lo, hi = expert_range
    T, K = topk_ids.shape
    flat = topk_ids.reshape(-1).to(torch.int64)
    keep = (flat >= lo) & (flat < hi)
    key = torch.where(keep, flat, torch.full_like(flat, 1 << 40))
    order = torch.sort(key, stable=True).indices
    m = int(keep.sum())
    idx = order[:m]
    counts = torch.bincount(flat[keep] - lo, minlength=hi - lo).to(torch.int64)
    tok = idx // K
    rows = x[tok]
    sc = scale[tok] if scale is not None else None
    return rows, idx.to(torch.int32), counts, sc


def moe_init_routing_v1(x: torch.Tensor, row_idx: torch.Tensor, topk_ids: torch.Tensor):
    """``npu_moe_init_routing(x, row_idx, expert_idx, active_num=T)`` followed by
    ``npu_moe_compute_expert_tokens`` (omni/quantization/compressed_tensors/
    compressed_tensors_moe.py:235-237).

    Returns (rows [T*K,H], expanded_src_to_dst_row int32 [T*K] indexed by
    row_idx value k*T+n, sorted expert ids int32 [T*K], cumulative expert token
    counts int64 [E] is computed by ``compute_expert_tokens``).
    """
    T, K = topk_ids.shape
    flat = topk_ids.reshape(-1).to(torch.int64)
    order = torch.sort(flat, stable=True).indices
    sorted_ids = flat[order]
    dst_to_src = row_idx.reshape(-1).to(torch.int64)[order]
    src_to_dst = torch.empty(T * K, dtype=torch.int64)
    src_to_dst[dst_to_src] = torch.arange(T * K)
    rows = x[dst_to_src % T]
    return rows, src_to_dst.to(torch.int32), sorted_ids.to(torch.int32)


def compute_expert_tokens(sorted_ids: torch.Tensor, num_experts: int) -> torch.Tensor:
    """``npu_moe_compute_expert_tokens``: cumulative count per expert
    (compressed_tensors_moe.py:237, consumed with group_list_type=0)."""
    return torch.cumsum(torch.bincount(sorted_ids.to(torch.int64), minlength=num_experts), 0)


# --------------------------------------------------------------------------
# Grouped int8 GEMMs and epilogues (C6, C7, C8)
# --------------------------------------------------------------------------
def _int_mm(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Exact int8 x int8 -> int32 matrix product."""
    if a.shape[0] == 0:
        return torch.zeros(0, b.shape[1], dtype=torch.int32)
    try:
        return torch._int_mm(a.contiguous(), b.contiguous())
    except Exception:
        return (a.double() @ b.double()).to(torch.int32)


def grouped_matmul_int32(a: torch.Tensor, w: torch.Tensor, counts: torch.Tensor) -> torch.Tensor:
    """``npu_grouped_matmul([a],[w],group_list=counts,group_list_type=1,
    output_dtype=int32)`` (fused_moe.py:531-533): rows are consecutive per
    group; acc[m,:] = a[m,:] . w[g(m)] exactly in int32.  w is [G, Kdim, N]."""
    out = torch.empty(a.shape[0], w.shape[2], dtype=torch.int32)
    start = 0
    for g, c in enumerate(counts.tolist()):
        if c:
            out[start:start + c] = _int_mm(a[start:start + c], w[g])
        start += c
    return out[:start] if start < a.shape[0] else out


def _group_of_rows(counts: torch.Tensor) -> torch.Tensor:
    return torch.repeat_interleave(torch.arange(counts.numel()), counts.to(torch.int64))


def dequant_swiglu_quant(acc: torch.Tensor, weight_scale: torch.Tensor, activation_scale: torch.Tensor,
                         counts: Optional[torch.Tensor], quant_scale: Optional[torch.Tensor] = None,
                         return_fp32: bool = False):
    """``npu_dequant_swiglu_quant(acc, weight_scale, activation_scale, bias=None,
    quant_scale, quant_offset=None, group_index=counts, activate_left=True,
    quant_mode=1)`` (fused_moe.py:534, :558-561, :675-677; activation.py:15-27).

    d = (float(acc) * weight_scale[g, n]) * activation_scale[m];
    y = silu(d[:, :I]) * d[:, I:]; y *= quant_scale[g] when given; then
    dynamic_quant(y).  weight_scale is [G, 2I] (or [2I] when counts is None).
    """
    m = acc.shape[0]
    if counts is None:
        ws = weight_scale.to(F32).reshape(1, -1).expand(m, -1)
        qs = None if quant_scale is None else quant_scale.to(F32).reshape(1, -1).expand(m, -1)
    else:
        g = _group_of_rows(counts)[:m]
        ws = weight_scale.to(F32)[g]
        qs = None if quant_scale is None else quant_scale.to(F32)[g]
    d = acc.to(F32) * ws
    d = d * activation_scale.to(F32).unsqueeze(-1)
    inter = d.shape[1] // 2
    y = silu_spec(d[:, :inter]) * d[:, inter:]
    if qs is not None:
        y = y * qs
    q, s = dynamic_quant(y)
    if return_fp32:
        return q, s, y
    return q, s


def grouped_matmul_dequant(a: torch.Tensor, w: torch.Tensor, w_scale: torch.Tensor, per_token_scale: torch.Tensor,
                           counts: torch.Tensor, out_dtype=torch.bfloat16) -> torch.Tensor:
    """``npu_grouped_matmul([a],[w],scale=[w_scale],per_token_scale=[s],
    output_dtype=bf16)`` (fused_moe.py:570-574, :681-685):
    o[m,:] = cast((float(acc[m,:]) * w_scale[g,:]) * s[m])."""
    acc = grouped_matmul_int32(a, w, counts)
    g = _group_of_rows(counts)[:acc.shape[0]]
    o = acc.to(F32) * w_scale.to(F32)[g]
    o = o * per_token_scale.to(F32)[:acc.shape[0]].unsqueeze(-1)
    return o.to(out_dtype)


# --------------------------------------------------------------------------
# Combine (C9)
# --------------------------------------------------------------------------
def grouped_matmul_finalize_routing(a: torch.Tensor, w: torch.Tensor, counts: torch.Tensor, w_scale: torch.Tensor,
                                    per_token_scale: torch.Tensor, shared_input: Optional[torch.Tensor],
                                    logit: torch.Tensor, row_index: torch.Tensor, output_bs: int,
                                    shared_input_weight: float = 1.0, shared_input_offset: int = 0,
                                    rows_bf16: bool = False) -> torch.Tensor:
    """``npu_grouped_matmul_finalize_routing`` (fused_moe.py:536).

    out[row_index[m], :] += logit[m] * ((float(acc2[m,:]) * w_scale[g,:]) * s[m])
    accumulated in fp32 in ascending m, starting from
    shared_input_weight * float(shared_input) on rows
    [offset, offset + shared_input.shape[0]).  Returns fp32 [output_bs, H].

    ``rows_bf16`` (the device library's bf16-row option, not a mode of the reference operator):
    every dequantised row is rounded to bf16 before it is weighted, which is what a bf16
    ``npu_grouped_matmul`` (fused_moe.py:570-574) hands to a finalize step.
    """
    acc = grouped_matmul_int32(a, w, counts)
    m = acc.shape[0]
    g = _group_of_rows(counts)[:m]
    v = acc.to(F32) * w_scale.to(F32)[g]
    v = v * per_token_scale.to(F32)[:m].unsqueeze(-1)
    if rows_bf16:
        v = v.to(torch.bfloat16).to(F32)
    v = logit.to(F32)[:m].unsqueeze(-1) * v
    out = torch.zeros(output_bs, w.shape[2], dtype=F32)
    if shared_input is not None:
        n = shared_input.shape[0]
        out[shared_input_offset:shared_input_offset + n] = shared_input.to(F32) * _c(shared_input_weight)
    _ordered_scatter_add(out, v, row_index[:m].to(torch.int64))
    return out


def _ordered_scatter_add(out: torch.Tensor, v: torch.Tensor, rows: torch.Tensor) -> None:
    """out[rows[m]] += v[m] for m ascending, one fp32 add per contribution."""
    m = v.shape[0]
    if m == 0:
        return
    order = torch.sort(rows, stable=True).indices       # group by token, ascending m inside
    r = rows[order]
    first = torch.ones(m, dtype=torch.bool)
    first[1:] = r[1:] != r[:-1]
    start = torch.nonzero(first).reshape(-1)
    seg = torch.cumsum(first.to(torch.int64), 0) - 1
    rank = torch.arange(m) - start[seg]
    for j in range(int(rank.max()) + 1):
        sel = rank == j
        out[r[sel]] = out[r[sel]] + v[order[sel]]


def moe_finalize_routing(rows: torch.Tensor, skip1: Optional[torch.Tensor], scales: torch.Tensor,
                         src_to_dst: torch.Tensor, drop_pad_mode: int = 0) -> torch.Tensor:
    """``npu_moe_finalize_routing(rows, skip1, None, None, scales,
    expanded_src_to_dst_row, ..., drop_pad_mode)``.

    out[n] = skip1[n] + sum_k scales[n,k] * rows[src_to_dst[idx(n,k)]], k
    ascending, fp32; idx = k*T + n for mode 0 (compressed_tensors_moe.py:
    252-254), idx = n*K + k for mode 2 (deepseek_moe.py:292-301).  A negative
    src_to_dst entry contributes nothing.  Output has the dtype of ``rows``.
    """
    T, K = scales.shape
    out = torch.zeros(T, rows.shape[1], dtype=F32) if skip1 is None else skip1.to(F32).clone()
    s2d = src_to_dst.to(torch.int64)
    n = torch.arange(T)
    for k in range(K):
        idx = k * T + n if drop_pad_mode == 0 else n * K + k
        dst = s2d[idx]
        ok = dst >= 0
        contrib = scales[:, k].to(F32).unsqueeze(-1) * rows[dst.clamp(min=0)].to(F32)
        out = torch.where(ok.unsqueeze(-1), out + contrib, out)
    return out.to(rows.dtype)


# --------------------------------------------------------------------------
# Dense W8A8 linear (shared expert, C10)
# --------------------------------------------------------------------------
def quant_matmul(x_int8: torch.Tensor, w: torch.Tensor, w_scale: torch.Tensor,
                 pertoken_scale: Optional[torch.Tensor], output_dtype) -> torch.Tensor:
    """``npu_quant_matmul`` (omni/quantization/compressed_tensors/schemes/
    compressed_tensors_w8a8_int8.py:101-109): raw int32 when output_dtype is
    int32, else cast((float(acc) * w_scale[n]) * pertoken_scale[m])."""
    acc = _int_mm(x_int8, w)
    if output_dtype == torch.int32:
        return acc
    o = acc.to(F32) * w_scale.to(F32).reshape(1, -1)
    if pertoken_scale is not None:
        o = o * pertoken_scale.to(F32).unsqueeze(-1)
    return o.to(output_dtype)


def shared_expert_mlp(x: torch.Tensor, w_gate_up: torch.Tensor, s_gate_up: torch.Tensor,
                      w_down: torch.Tensor, s_down: torch.Tensor, return_stages: bool = False):
    """``ReplicatedDeepseekMLP.forward`` on the W8A8 scheme
    (omni/models/common/layers/moe/deepseek_moe.py:100-118; activation.py:15-27;
    compressed_tensors_w8a8_int8.py:84-110).  w_gate_up [H,2I], w_down [I,H]."""
    xq, xs = dynamic_quant(x)
    acc = quant_matmul(xq, w_gate_up, s_gate_up, None, torch.int32)
    hq, hs = dequant_swiglu_quant(acc, s_gate_up, xs, None)
    out = quant_matmul(hq, w_down, s_down, hs, torch.bfloat16)
    if return_stages:
        return out, dict(x_q=xq, x_s=xs, acc1=acc, h_q=hq, h_s=hs)
    return out


# --------------------------------------------------------------------------
# Pipelines
# --------------------------------------------------------------------------
def fused_experts_w8a8_allgather_ep(x_int8, pertoken_scale, w1, w2, w1_scale, w2_scale, topk_weights, topk_ids,
                                    expert_range, shared_input=None, return_stages=False, rows_bf16=False):
    """``fused_experts_w8a8_allgather_ep`` (fused_moe.py:489-538): the local-share
    pipeline.  x_int8 [T,H]; w1 [E_loc,H,2I]; w2 [E_loc,I,H]; topk_ids are
    global ids; only ids in expert_range = [lo, hi) are computed here.
    The reference passes zeros as shared_input (fused_moe.py:521)."""
    T, K = topk_ids.shape
    rows, idx, counts, scale = moe_init_routing_v2(x_int8, topk_ids, pertoken_scale, expert_range)
    w_sorted = topk_weights.reshape(-1)[idx.to(torch.int64)]
    row_index = (idx // K).to(torch.int64)
    acc1 = grouped_matmul_int32(rows, w1, counts)
    hq, hs, y = dequant_swiglu_quant(acc1, w1_scale, scale, counts,
                                     quant_scale=torch.ones(w1.shape[0], w1_scale.shape[-1] // 2), return_fp32=True)
    if shared_input is None:
        shared_input = torch.zeros(T, w2.shape[2], dtype=torch.bfloat16)
    out32 = grouped_matmul_finalize_routing(hq, w2, counts, w2_scale.float(), hs, shared_input, w_sorted,
                                            row_index, T, rows_bf16=rows_bf16)
    out = out32.to(torch.bfloat16)
    if return_stages:
        acc2 = grouped_matmul_int32(hq, w2, counts)
        return out, dict(idx=idx, counts=counts, rows=rows, row_scale=scale, acc1=acc1, y=y, h_q=hq, h_s=hs,
                         acc2=acc2, out32=out32)
    return out


def fused_experts_w8a8_allgather_ep_a2(x_int8, pertoken_scale, w1, w2, w1_scale, w2_scale, topk_weights, topk_ids,
                                       expert_range, smooth_scale, pd_seperate_prefill=False, return_stages=False):
    """``fused_experts_w8a8_allgather_ep_a2`` (fused_moe.py:844-937): the local-share pipeline of the A2 platform
    branch.  As ``fused_experts_w8a8_allgather_ep`` with ``quant_scale=smooth_scale`` ([E_loc, I] fp32) inside
    ``npu_dequant_swiglu_quant`` (:907), and two tails:

    * default (:919-927): ``npu_grouped_matmul_finalize_routing`` on fp32 sums with a zero shared input;
    * ``pd_seperate_prefill`` (:909-918): ``npu_grouped_matmul(..., output_dtype=bf16)`` with the bf16 ``w2_scale``
      that ``process_weights_after_loading`` makes under that flag (compressed_tensors_moe.py:100-101), then
      ``npu_moe_finalize_routing(rows, None, None, None, topk_weights.to(bf16), expanded_x_idx, topk_ids,
      drop_pad_mode=3)`` with the source-to-slot index that ``row_idx_type=0`` asks of the sort (:868):
      out[n] = sum_k float(bf16(w[n,k])) * float(rows[slot(n*K+k)]) over the kept assignments, k ascending, fp32,
      rounded to bf16.  (What mode 3 does with a dropped assignment is not observable here: it contributes nothing.)

    The index patch-up of :879-884 only rewrites entries past the kept total, which nothing reads.
    """
    T, K = topk_ids.shape
    rows, idx, counts, scale = moe_init_routing_v2(x_int8, topk_ids, pertoken_scale, expert_range)
    acc1 = grouped_matmul_int32(rows, w1, counts)
    hq, hs, y = dequant_swiglu_quant(acc1, w1_scale, scale, counts, quant_scale=smooth_scale, return_fp32=True)
    if pd_seperate_prefill:
        out_rows = grouped_matmul_dequant(hq, w2, w2_scale.to(torch.bfloat16), hs, counts, out_dtype=torch.bfloat16)
        src_to_dst = torch.full((T * K,), -1, dtype=torch.int32)
        src_to_dst[idx.to(torch.int64)] = torch.arange(idx.numel(), dtype=torch.int32)
        out = moe_finalize_routing(out_rows, None, topk_weights.to(torch.bfloat16), src_to_dst, drop_pad_mode=2)
    else:
        w_sorted = topk_weights.reshape(-1)[idx.to(torch.int64)]
        row_index = (idx // K).to(torch.int64)
        shared_input = torch.zeros(T, w2.shape[2], dtype=torch.bfloat16)
        out = grouped_matmul_finalize_routing(hq, w2, counts, w2_scale.float(), hs, shared_input, w_sorted, row_index,
                                              T).to(torch.bfloat16)
    if return_stages:
        return out, dict(idx=idx, counts=counts, y=y, h_q=hq, h_s=hs)
    return out


def moe_expert_quant_forward(rows_int8, w1, w2, w1_scale, w2_scale, counts, dynamic_scale,
                             w2_scale_bf16: bool = False):
    """``moe_expert_quant_farword`` with quant_mode != 0 / ``gmm_expert``
    (fused_moe.py:541-575, 663-687): rows are already grouped by local expert."""
    acc1 = grouped_matmul_int32(rows_int8, w1, counts)
    hq, hs = dequant_swiglu_quant(acc1, w1_scale, dynamic_scale, counts,
                                  quant_scale=torch.ones(w1.shape[0], w1_scale.shape[-1] // 2))
    ws2 = w2_scale.to(torch.bfloat16) if w2_scale_bf16 else w2_scale
    return grouped_matmul_dequant(hq, w2, ws2, hs, counts, torch.bfloat16)


def swiglu_bf16(x: torch.Tensor) -> torch.Tensor:
    """``npu_swiglu`` on bf16 (compressed_tensors_moe.py:246): computed in fp32
    from the bf16 inputs, one rounding to bf16 at the end."""
    inter = x.shape[-1] // 2
    xf = x.to(F32)
    return (silu_spec(xf[..., :inter]) * xf[..., inter:]).to(x.dtype)


def fused_experts_w8a8(hidden_states, w1, w2, w1_scale, w2_scale, topk_weights, topk_ids, row_idx,
                       return_stages=False):
    """``fused_experts_w8a8`` (compressed_tensors_moe.py:221-254): the non-EP
    pipeline with bf16 between the stages.  hidden_states bf16 [T,H]."""
    T, _ = hidden_states.shape
    E = w1.shape[0]
    rows, src_to_dst, sorted_ids = moe_init_routing_v1(hidden_states, row_idx, topk_ids)
    cum = compute_expert_tokens(sorted_ids, E)
    counts = torch.diff(cum, prepend=torch.zeros(1, dtype=cum.dtype))
    act_dtype = hidden_states.dtype
    s1 = w1_scale.to(torch.bfloat16)
    s2 = w2_scale.to(torch.bfloat16)
    xq, xs = dynamic_quant(rows)
    gate_up = grouped_matmul_dequant(xq, w1, s1, xs, counts, act_dtype)
    act = swiglu_bf16(gate_up)
    hq, hs = dynamic_quant(act)
    rows_out = grouped_matmul_dequant(hq, w2, s2, hs, counts, act_dtype).float()
    out = moe_finalize_routing(rows_out, None, topk_weights, src_to_dst, drop_pad_mode=0).to(torch.bfloat16)
    if return_stages:
        return out, dict(src_to_dst=src_to_dst, counts=counts, x_q=xq, x_s=xs, gate_up=gate_up, h_q=hq, h_s=hs,
                         rows_out=rows_out)
    return out


def deepseek_moe_forward(x, logits, bias, routed, shared, top_k, n_group, topk_group, scale, expert_range,
                         return_stages=False):
    """``DeepseekMoE._forward_{prefill,decode}_norm`` on one device without
    collectives (deepseek_moe.py:243-368): shared expert, dynamic quant,
    noaux_tc routing, local-share experts, plus the shared output.

    routed = (w1, w1_scale, w2, w2_scale); shared = (w_gate_up, s_gate_up,
    w_down, s_down) or None."""
    shared_out = shared_expert_mlp(x, *shared) if shared is not None else None
    xq, xs = dynamic_quant(x)
    w, ids = route_noaux_tc(logits, bias, top_k, n_group, topk_group, scale)
    w1, s1, w2, s2 = routed
    res = fused_experts_w8a8_allgather_ep(xq, xs, w1, w2, s1, s2, w, ids, expert_range, return_stages=return_stages)
    out, st = res if return_stages else (res, None)
    if shared_out is not None:
        out = out + shared_out
    if return_stages:
        st.update(topk_w=w, topk_ids=ids, x_q=xq, x_s=xs, shared_out=shared_out)
        return out, st
    return out


# --------------------------------------------------------------------------
# Independent witness: dense brute force without any permutation
# --------------------------------------------------------------------------
def dense_bruteforce(x_int8, pertoken_scale, w1, w2, w1_scale, w2_scale, topk_weights, topk_ids, expert_range):
    """Every token through every local expert it selected, one expert at a time
    on the full token batch, in float64 after the exact integer products.
    Independent of the sort / scatter index logic.  Returns float64 [T,H]."""
    lo, hi = expert_range
    T = x_int8.shape[0]
    out = torch.zeros(T, w2.shape[2], dtype=torch.float64)
    for e in range(lo, hi):
        sel = (topk_ids == e)
        tok = sel.any(dim=1)
        if not bool(tok.any()):
            continue
        wt = (topk_weights.double() * sel).sum(dim=1)[tok]
        a = x_int8[tok]
        acc = _int_mm(a, w1[e - lo]).double()
        d = acc * w1_scale[e - lo].double() * pertoken_scale[tok].double().unsqueeze(-1)
        inter = d.shape[1] // 2
        y = d[:, :inter] / (1.0 + torch.exp(-d[:, :inter])) * d[:, inter:]
        s = y.abs().amax(dim=1) / 127.0
        q = torch.round(y / torch.where(s > 0, s, torch.ones_like(s)).unsqueeze(-1)).clamp(-128, 127)
        o = (q @ w2[e - lo].double()) * w2_scale[e - lo].double() * s.unsqueeze(-1)
        out[tok] += wt.unsqueeze(-1) * o
    return out


# --------------------------------------------------------------------------
# Synthetic inputs of the benchmark configurations
# --------------------------------------------------------------------------
def quantize_weight_per_channel(w_fp32: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Symmetric per-output-channel int8: w_fp32 is [out, in]; s = absmax over
    the input dim / 127; q = round(w / s).  Returns (q int8 [out,in], s fp32 [out])."""
    s = w_fp32.abs().amax(dim=1) / 127.0
    s = torch.where(s > 0, s, torch.ones_like(s))
    q = torch.round(w_fp32 / s.unsqueeze(1)).clamp(-127, 127).to(torch.int8)
    return q, s.to(F32)


def make_expert_weights(num_experts: int, hidden: int, inter: int, gen: torch.Generator, std: float = 0.02):
    """Checkpoint-layout weights as ``create_weights`` declares them
    (compressed_tensors_moe.py:44-92): w13 int8 [E, 2I, H] (w1/gate rows first,
    w3/up rows second), w2 int8 [E, H, I], scales fp32 [E, 2I] / [E, H]."""
    w13 = torch.empty(num_experts, 2 * inter, hidden, dtype=torch.int8)
    w2 = torch.empty(num_experts, hidden, inter, dtype=torch.int8)
    s13 = torch.empty(num_experts, 2 * inter, dtype=F32)
    s2 = torch.empty(num_experts, hidden, dtype=F32)
    for e in range(num_experts):
        q, s = quantize_weight_per_channel(torch.randn(2 * inter, hidden, generator=gen) * std)
        w13[e], s13[e] = q, s
        q, s = quantize_weight_per_channel(torch.randn(hidden, inter, generator=gen) * std)
        w2[e], s2[e] = q, s
    return w13, s13, w2, s2


def local_dense_ids(T: int, K: int, n_local: int, gen: torch.Generator, lo: int = 0) -> torch.Tensor:
    """Each token picks K distinct local experts uniformly at random."""
    perm = torch.rand(T, n_local, generator=gen).argsort(dim=1)[:, :K]
    return (perm + lo).to(torch.int32)


def zipf_logit_offsets(n_local: int, gen: torch.Generator, s: float = 1.2, n_empty: int = 4) -> torch.Tensor:
    """log of a Zipf(s) pmf over a seeded permutation of the local experts; the
    ``n_empty`` least popular ones get -inf so they receive no token."""
    ranks = torch.arange(1, n_local + 1, dtype=torch.float64)
    pmf = ranks.pow(-s)
    pmf = pmf / pmf.sum()
    off = pmf.log().to(F32)
    off[n_local - n_empty:] = float("-inf")
    perm = torch.randperm(n_local, generator=gen)
    out = torch.empty(n_local, dtype=F32)
    out[perm] = off
    return out
