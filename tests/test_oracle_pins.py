"""Pins of the CPU oracle against evidence that does not come from the oracle's own formulas:
library routines (torch, transformers' DeepseekV3TopkRouter, numpy), the reference's own pure-torch
routing code restated side by side, closed-form invariants, brute force on tiny inputs, and an
end-to-end dense witness in float64.  The reference holds no golden vector for this path, so these
pins (and the fixtures under tests/golden, which freeze the oracle's outputs) are what parity rests on."""
import itertools
import os
import types

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tests.helpers import Layer, cosine, gen, rel_err, tokens


def ulp_diff(a, b):
    ai = a.contiguous().view(torch.int32).long()
    bi = b.contiguous().view(torch.int32).long()
    ai = torch.where(ai < 0, -(ai & 0x7fffffff), ai)
    bi = torch.where(bi < 0, -(bi & 0x7fffffff), bi)
    return (ai - bi).abs()


# ------------------------------------------------------------------ transcendental
def test_exp_spec_against_libm():
    x = torch.linspace(-86.9, 86.9, 1_000_001)
    got = O.exp_spec(x)
    want = torch.exp(x.double()).float()
    assert int(ulp_diff(got, want).max()) <= 2
    assert float(O.exp_spec(torch.tensor([0.0]))) == 1.0
    assert bool((got[1:] >= got[:-1]).all()), "exp must be monotone"
    # clamping: finite, positive, normal numbers at both ends
    ends = O.exp_spec(torch.tensor([-1e4, -87.0, 87.0, 1e4, float("inf"), float("-inf")]))
    assert bool(torch.isfinite(ends).all()) and bool((ends >= torch.finfo(torch.float32).tiny).all())


def test_sigmoid_silu_spec_against_torch():
    x = torch.cat([torch.linspace(-30, 30, 600_001), torch.randn(100_000, generator=gen(0)) * 4])
    s = O.sigmoid_spec(x)
    assert float((s.double() - torch.sigmoid(x.double())).abs().max()) < 1.5e-7
    y = O.silu_spec(x)
    ref = torch.nn.functional.silu(x.double())
    assert float((y.double() - ref).abs().max()) < 2e-6
    nz = ref.abs() > 1e-30
    assert float(((y.double() - ref)[nz] / ref[nz]).abs().max()) < 4e-7      # ~3 ulp
    assert float(O.silu_spec(torch.tensor([0.0]))) == 0.0
    assert float(O.sigmoid_spec(torch.tensor([0.0]))) == 0.5


# ------------------------------------------------------------------ routing
def _hf_router(E, K, n_group, topk_group, scale, bias):
    from transformers.models.deepseek_v3.modeling_deepseek_v3 import DeepseekV3TopkRouter
    cfg = types.SimpleNamespace(num_experts_per_tok=K, num_local_experts=E, hidden_size=E, routed_scaling_factor=scale,
                                n_group=n_group, topk_group=topk_group, norm_topk_prob=True)
    r = DeepseekV3TopkRouter(cfg)
    with torch.no_grad():
        r.weight.copy_(torch.eye(E))            # logits = input, exactly
        r.e_score_correction_bias.copy_(bias)
    return r


@pytest.mark.parametrize("T,E,ng,tg,K", [(512, 256, 8, 4, 8), (64, 64, 4, 2, 6), (33, 32, 8, 4, 8)])
def test_route_noaux_tc_against_transformers(T, E, ng, tg, K):
    g = gen(1)
    logits = torch.randn(T, E, generator=g) * 2
    bias = torch.randn(E, generator=g) * 0.01
    w, ids = O.route_noaux_tc(logits, bias, K, ng, tg, 2.5)
    with torch.no_grad():
        lg, hw, hi = _hf_router(E, K, ng, tg, 2.5, bias)(logits)
    assert torch.equal(lg, logits)
    dense = torch.zeros(T, E).scatter_(1, ids.long(), w)
    hdense = torch.zeros(T, E).scatter_(1, hi, hw)
    assert bool(((dense != 0) == (hdense != 0)).all()), "selected expert sets differ from the library router"
    assert float((dense - hdense).abs().max()) < 1e-6
    # invariants
    assert all(len(set(r.tolist())) == K for r in ids)
    groups = ids // (E // ng)
    assert all(len(set(r.tolist())) <= tg for r in groups)
    assert float((w.sum(-1) - 2.5).abs().max()) < 1e-5
    c = torch.sigmoid(logits) + bias
    picked = torch.gather(c, 1, ids.long())
    assert bool((picked[:, :-1] >= picked[:, 1:] - 1e-7).all()), "output must be in descending score"


def test_route_noaux_tc_bruteforce_tiny():
    """E=8, 4 groups of 2, keep 2 groups, top-2: enumerate every pair of groups and of experts."""
    g = gen(2)
    logits = torch.randn(200, 8, generator=g)
    bias = torch.randn(8, generator=g) * 0.1
    w, ids = O.route_noaux_tc(logits, bias, 2, 4, 2, 1.0)
    s = O.sigmoid_spec(logits)
    c = (s + bias).tolist()
    for t in range(200):
        gs = [c[t][2 * i] + c[t][2 * i + 1] for i in range(4)]
        best_groups = max(itertools.combinations(range(4), 2), key=lambda p: (gs[p[0]] + gs[p[1]], -p[0], -p[1]))
        cand = [2 * gi + j for gi in best_groups for j in range(2)]
        best = sorted(cand, key=lambda e: (-c[t][e], e))[:2]
        assert ids[t].tolist() == best


def _reference_grouped_topk(gating_output, topk, renormalize, num_expert_group, topk_group, scoring_func, bias):
    """fused_moe.py:38-84 restated line by line with torch's own softmax / sigmoid / topk."""
    gating_output = gating_output.float()
    scores = torch.softmax(gating_output, dim=-1) if scoring_func == "softmax" else gating_output.sigmoid()
    if bias is not None:
        scores = scores + bias.unsqueeze(0)
    num_token = scores.shape[0]
    group_scores = scores.view(num_token, num_expert_group, -1).max(dim=-1).values
    group_idx = torch.topk(group_scores, k=topk_group, dim=-1, sorted=False)[1]
    group_mask = torch.zeros_like(group_scores)
    group_mask.scatter_(1, group_idx, 1)
    score_mask = group_mask.unsqueeze(-1).expand(num_token, num_expert_group,
                                                 scores.shape[-1] // num_expert_group).reshape(num_token, -1)
    tmp_scores = scores.masked_fill(~score_mask.bool(), 0.0)
    topk_weights, topk_ids = torch.topk(tmp_scores, k=topk, dim=-1, sorted=False)
    if renormalize:
        topk_weights = topk_weights / topk_weights.sum(dim=-1, keepdim=True)
    return topk_weights, topk_ids.int()


@pytest.mark.parametrize("scoring,with_bias", [("softmax", False), ("sigmoid", False), ("sigmoid", True)])
def test_route_grouped_topk_against_reference_torch_code(scoring, with_bias):
    g = gen(3)
    logits = torch.randn(300, 256, generator=g)
    bias = torch.randn(256, generator=g) * 0.01 if with_bias else None
    w, ids, row = O.route_grouped_topk(logits, 8, True, 8, 4, scoring, bias)
    rw, rid = _reference_grouped_topk(logits, 8, True, 8, 4, scoring, bias)
    a = torch.zeros(300, 256).scatter_(1, ids.long(), w)
    b = torch.zeros(300, 256).scatter_(1, rid.long(), rw)
    assert bool(((a != 0) == (b != 0)).all())
    assert float((a - b).abs().max()) < 1e-6
    assert row[5, 3] == 3 * 300 + 5


def test_route_softmax_topk_against_torch():
    logits = torch.randn(128, 8, generator=gen(4)) * 3
    for renorm in (True, False):
        w, ids, row = O.route_softmax_topk(logits, 2, renorm)
        p = torch.softmax(logits, -1)
        tw, ti = p.topk(2)
        if renorm:
            tw = tw / tw.sum(-1, keepdim=True)
        assert torch.equal(ids.long(), ti)
        assert float((w - tw).abs().max()) < 3e-7
    assert float((O.softmax_spec(torch.randn(7, 300, generator=gen(5))).sum(-1) - 1).abs().max()) < 1e-6


# ------------------------------------------------------------------ dynamic quant
def test_dynamic_quant_invariants_and_numpy():
    x = tokens(64, 7168, 6, outlier_frac=0.001)
    x[3] = 0
    q, s = O.dynamic_quant(x)
    xf = x.float()
    nz = s > 0
    assert int(q[3].abs().max()) == 0 and float(s[3]) == 0.0
    assert bool((q[nz].abs().amax(dim=1) == 127).all())
    assert bool(((xf - q.float() * s.unsqueeze(1)).abs() <= s.unsqueeze(1) * 0.5 * (1 + 1e-6)).all())
    # float32 numpy recomputation with a true division and round-half-even
    xn = xf.numpy()
    sn = (np.abs(xn).max(axis=1) / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        qn = np.where(sn[:, None] > 0, np.rint(xn / np.where(sn > 0, sn, 1)[:, None]), 0).clip(-128, 127)
    assert np.array_equal(sn, s.numpy()) and np.array_equal(qn.astype(np.int8), q.numpy())
    # idempotence: quantising the dequantised tensor gives the same integers
    q2, s2 = O.dynamic_quant(q.float() * s.unsqueeze(1))
    assert torch.equal(q2, q)
    # half-way cases round to even
    h = torch.tensor([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5]])
    assert O.dynamic_quant(h)[0].tolist() == [[127, 0, 2, 2, 0, -2]]


# ------------------------------------------------------------------ permutation
def test_init_routing_v2_invariants():
    g = gen(7)
    T, K, E, lo, hi = 300, 8, 256, 64, 96
    ids = torch.rand(T, E, generator=g).argsort(1)[:, :K].int()
    x = torch.randint(-128, 128, (T, 16), generator=g, dtype=torch.int8)
    sc = torch.rand(T, generator=g)
    rows, idx, counts, scg = O.moe_init_routing_v2(x, ids, sc, (lo, hi))
    flat = ids.reshape(-1).numpy()
    keep = (flat >= lo) & (flat < hi)
    order = np.argsort(np.where(keep, flat, 1 << 30), kind="stable")[:keep.sum()]
    assert np.array_equal(idx.numpy(), order)
    assert np.array_equal(counts.numpy(), np.bincount(flat[keep] - lo, minlength=hi - lo))
    e_sorted = flat[idx.numpy()]
    assert bool((np.diff(e_sorted) >= 0).all())
    assert torch.equal(rows, x[idx.long() // K]) and torch.equal(scg, sc[idx.long() // K])


def test_init_routing_v1_roundtrip():
    g = gen(8)
    T, K, E = 100, 2, 8
    ids = torch.rand(T, E, generator=g).argsort(1)[:, :K].int()
    x = torch.randn(T, 8, generator=g)
    row_idx = torch.arange(T * K, dtype=torch.int32).view(K, T).t().contiguous()
    rows, s2d, sid = O.moe_init_routing_v1(x, row_idx, ids)
    assert sorted(s2d.tolist()) == list(range(T * K))
    for n in (0, 17, 99):
        for k in range(K):
            d = int(s2d[k * T + n])
            assert torch.equal(rows[d], x[n]) and int(sid[d]) == int(ids[n, k])
    assert O.compute_expert_tokens(sid, E).tolist() == np.cumsum(np.bincount(ids.reshape(-1).numpy(), minlength=E)).tolist()


# ------------------------------------------------------------------ GEMMs, epilogues, combine
def test_grouped_matmul_int32_against_fp64():
    g = gen(9)
    a = torch.randint(-128, 128, (40, 7168), generator=g, dtype=torch.int8)
    w = torch.randint(-128, 128, (3, 7168, 64), generator=g, dtype=torch.int8)
    counts = torch.tensor([17, 0, 23])
    acc = O.grouped_matmul_int32(a, w, counts)
    ref = torch.cat([a[:17].double() @ w[0].double(), a[17:].double() @ w[2].double()])
    assert torch.equal(acc.double(), ref)
    assert int(acc.abs().max()) < 2 ** 31


def test_dequant_swiglu_quant_closed_form():
    g = gen(10)
    acc = torch.randint(-200000, 200000, (50, 256), generator=g, dtype=torch.int32)
    ws = torch.rand(2, 256, generator=g) * 1e-3
    ts = torch.rand(50, generator=g) * 0.05
    counts = torch.tensor([20, 30])
    q, s, y = O.dequant_swiglu_quant(acc, ws, ts, counts, return_fp32=True)
    grp = torch.repeat_interleave(torch.arange(2), counts)
    d = acc.double() * ws.double()[grp] * ts.double().unsqueeze(1)
    yd = d[:, :128] / (1 + torch.exp(-d[:, :128])) * d[:, 128:]
    assert rel_err(y, yd) < 1e-6
    assert float((s.double() - yd.abs().amax(1) / 127).abs().max() / s.max()) < 1e-6
    # gate is the first half, up the second: swapping halves must change the result
    acc_sw = torch.cat([acc[:, 128:], acc[:, :128]], 1)
    ws_sw = torch.cat([ws[:, 128:], ws[:, :128]], 1)
    y_sw = O.dequant_swiglu_quant(acc_sw, ws_sw, ts, counts, return_fp32=True)[2]
    assert not torch.allclose(y, y_sw)
    # group_index=None form (dense linear) equals a single group
    q1, s1 = O.dequant_swiglu_quant(acc, ws[0], ts, None)
    q2, s2 = O.dequant_swiglu_quant(acc, ws[:1], ts, torch.tensor([50]))
    assert torch.equal(q1, q2) and torch.equal(s1, s2)


def test_finalize_routing_forms():
    g = gen(11)
    T, K, H = 20, 3, 32
    rows = torch.randn(T * K, H, generator=g)
    w = torch.rand(T, K, generator=g)
    skip = torch.randn(T, H, generator=g)
    s2d = torch.randperm(T * K, generator=g).int()
    out0 = O.moe_finalize_routing(rows, skip, w, s2d, 0)
    out2 = O.moe_finalize_routing(rows, skip, w, s2d, 2)
    n = torch.arange(T)
    ref0 = skip.double() + sum(w[:, k].double().unsqueeze(1) * rows[s2d[k * T + n].long()].double() for k in range(K))
    ref2 = skip.double() + sum(w[:, k].double().unsqueeze(1) * rows[s2d[n * K + k].long()].double() for k in range(K))
    assert rel_err(out0, ref0) < 1e-6 and rel_err(out2, ref2) < 1e-6
    assert not torch.allclose(out0, out2)


@pytest.mark.parametrize("T,K,n_local,E,H,I", [(64, 2, 8, 8, 1024, 512), (40, 8, 4, 32, 512, 256)])
def test_pipeline_against_dense_bruteforce(T, K, n_local, E, H, I):
    """The sorted / grouped / scattered pipeline equals the permutation-free dense computation."""
    lay = Layer(n_local, H, I, seed=12)
    g = gen(13)
    x = tokens(T, H, 13)
    xq, xs = O.dynamic_quant(x)
    ids = torch.rand(T, E, generator=g).argsort(1)[:, :K].int()
    w = torch.rand(T, K, generator=g)
    lo = 0 if E == n_local else 8
    out, st = O.fused_experts_w8a8_allgather_ep(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, (lo, lo + n_local),
                                                return_stages=True)
    brute = O.dense_bruteforce(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, (lo, lo + n_local))
    assert rel_err(st["out32"], brute) < 2e-3          # int8 rounding flips between fp32 and fp64 SwiGLU
    assert rel_err(out.float(), brute) < 5e-3
    # and the non-EP pipeline (bf16 between stages) stays close to the same dense result
    if E == n_local:
        row_idx = torch.arange(T * K, dtype=torch.int32).view(K, T).t().contiguous()
        out_u = O.fused_experts_w8a8(x, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, row_idx)
        assert rel_err(out_u.float(), brute) < 2e-2


def test_shared_expert_against_float_mlp():
    lay = Layer(1, 1024, 512, seed=14, shared=True)
    x = tokens(32, 1024, 14)
    out = O.shared_expert_mlp(x, *lay.shared)
    wgu = lay.shared[0].double() * lay.shared[1].double().unsqueeze(0)
    wd = lay.shared[2].double() * lay.shared[3].double().unsqueeze(0)
    h = x.double() @ wgu
    y = torch.nn.functional.silu(h[:, :512]) * h[:, 512:]
    assert rel_err(out.float(), y @ wd) < 4e-2           # noise of two int8 quantisations of the activations
    assert cosine(out.float(), y @ wd) > 0.999


# ------------------------------------------------------------------ golden fixtures
def test_golden_fixtures_reproduce():
    """tests/golden/*.pt freeze the oracle's outputs on the toy configuration (made by
    tests/golden/make_golden.py); a change of the oracle's arithmetic shows up here."""
    from tests.golden import make_golden
    path = os.path.join(os.path.dirname(__file__), "golden", "toy_config1.pt")
    saved = torch.load(path, weights_only=True)
    fresh = make_golden.toy_config1()
    assert sorted(saved) == sorted(fresh)
    for k in saved:
        assert torch.equal(saved[k], fresh[k]), k


# ------------------------------------------------------------------ direct pins of the dequantising GEMMs and bf16 SwiGLU
def _bf16_steps(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Distance in bf16 representable steps between two bf16 tensors."""
    ai = a.contiguous().view(torch.int16).to(torch.int32)
    bi = b.contiguous().view(torch.int16).to(torch.int32)
    ai = torch.where(ai < 0, -(ai & 0x7fff), ai)
    bi = torch.where(bi < 0, -(bi & 0x7fff), bi)
    return (ai - bi).abs()


def test_grouped_matmul_dequant_closed_form():
    """o[m] = (acc[m] . w_scale[g(m)]) . s[m] in fp64 from the exact integer product: a wrong group's
    scale, a missing per-token scale or a transposed weight must fail."""
    g = gen(20)
    K, N = 512, 96
    a = torch.randint(-128, 128, (45, K), generator=g, dtype=torch.int8)
    w = torch.randint(-128, 128, (4, K, N), generator=g, dtype=torch.int8)
    ws = torch.rand(4, N, generator=g) * 1e-3 + 1e-4
    ts = torch.rand(45, generator=g) * 0.05 + 0.01
    counts = torch.tensor([11, 0, 30, 4])
    grp = torch.repeat_interleave(torch.arange(4), counts)
    exact = torch.stack([a[m].double() @ w[grp[m]].double() for m in range(45)])
    want = exact * ws.double()[grp] * ts.double().unsqueeze(1)
    got32 = O.grouped_matmul_dequant(a, w, ws, ts, counts, torch.float32)
    assert float(((got32.double() - want) / want.abs().clamp(min=1e-30)).abs().max()) < 3e-7   # two fp32 roundings
    got16 = O.grouped_matmul_dequant(a, w, ws, ts, counts, torch.bfloat16)
    assert int(_bf16_steps(got16, want.to(torch.bfloat16)).max()) <= 1
    assert float((_bf16_steps(got16, want.to(torch.bfloat16)) == 0).float().mean()) > 0.99
    # the mistakes this must catch
    wrong_group = exact * ws.double()[(grp + 1) % 4] * ts.double().unsqueeze(1)
    no_token_scale = exact * ws.double()[grp]
    for bad in (wrong_group, no_token_scale):
        assert rel_err(got32, bad) > 0.1
    # rows of an empty group do not exist: 45 rows, group 1 contributes none
    assert got32.shape == (45, N)


def test_quant_matmul_closed_form():
    g = gen(21)
    x = torch.randint(-128, 128, (33, 256), generator=g, dtype=torch.int8)
    w = torch.randint(-128, 128, (256, 80), generator=g, dtype=torch.int8)
    ws = torch.rand(80, generator=g) * 1e-3 + 1e-4
    ts = torch.rand(33, generator=g) * 0.05 + 0.01
    exact = x.double() @ w.double()
    assert torch.equal(O.quant_matmul(x, w, ws, None, torch.int32).double(), exact)
    got = O.quant_matmul(x, w, ws, ts, torch.bfloat16)
    want = (exact * ws.double() * ts.double().unsqueeze(1)).to(torch.bfloat16)
    assert int(_bf16_steps(got, want).max()) <= 1 and float((_bf16_steps(got, want) == 0).float().mean()) > 0.99
    got_nots = O.quant_matmul(x, w, ws, None, torch.float32)
    assert rel_err(got_nots, exact * ws.double()) < 1e-6
    assert rel_err(got.float(), exact * ws.double()) > 0.1          # the per-token scale is applied
    assert rel_err(got.float(), (x.double() @ w.double().flip(0)) * ws.double() * ts.double().unsqueeze(1)) > 0.1


def test_swiglu_bf16_closed_form():
    g = gen(22)
    x = (torch.randn(64, 512, generator=g) * 3).to(torch.bfloat16)
    got = O.swiglu_bf16(x)
    xd = x.double()
    want = (xd[:, :256] / (1 + torch.exp(-xd[:, :256])) * xd[:, 256:])
    steps = _bf16_steps(got, want.to(torch.bfloat16))
    assert int(steps.max()) <= 1 and float((steps == 0).float().mean()) > 0.99   # one rounding at the end
    swapped = (xd[:, 256:] / (1 + torch.exp(-xd[:, 256:])) * xd[:, :256])
    assert rel_err(got.float(), swapped) > 0.1                                   # gate is the first half
    assert got.dtype == torch.bfloat16 and got.shape == (64, 256)


# ------------------------------------------------------------------ pipelines: grouped-rows form and the whole block
def _fp64_expert_rows(rows_q, row_scale, w1, s1, w2, s2, counts):
    """Permutation-free fp64 witness of the grouped-rows pipeline: one expert at a time, exact integer
    products, SwiGLU and both quantisation steps in float64.  Returns (rows fp64 [M,H], y fp64)."""
    M = rows_q.shape[0]
    out = torch.zeros(M, w2.shape[2], dtype=torch.float64)
    ys = torch.zeros(M, w1.shape[2] // 2, dtype=torch.float64)
    start = 0
    for e, c in enumerate(counts.tolist()):
        if c == 0:
            continue
        sl = slice(start, start + c)
        d = (rows_q[sl].double() @ w1[e].double()) * s1[e].double() * row_scale[sl].double().unsqueeze(1)
        inter = d.shape[1] // 2
        y = d[:, :inter] / (1 + torch.exp(-d[:, :inter])) * d[:, inter:]
        s = y.abs().amax(1) / 127.0
        q = torch.round(y / torch.where(s > 0, s, torch.ones_like(s)).unsqueeze(1)).clamp(-128, 127)
        out[sl] = (q @ w2[e].double()) * s2[e].double() * s.unsqueeze(1)
        ys[sl] = y
        start += c
    return out, ys


@pytest.mark.parametrize("bf16_scale", [False, True])
def test_moe_expert_quant_forward_against_fp64_witness(bf16_scale):
    """moe_expert_quant_farword / gmm_expert (fused_moe.py:541-575, 663-687): rows grouped by expert.
    (a) whole pipeline against the fp64 witness (int8 rounding flips bound the agreement);
    (b) the second stage alone, fed the oracle's own int8 rows, must land within one bf16 step of the
    fp64 closed form *with the w2 scale it was asked to use*: a skipped (or unasked-for) bf16 rounding of
    the scale moves the rows by ~2^-9 and fails;  (c) wrong group boundaries fail."""
    lay = Layer(5, 512, 256, seed=30)
    g = gen(31)
    counts = torch.tensor([9, 0, 23, 1, 14])
    M = int(counts.sum())
    x = tokens(M, 512, 31)
    rows_q, rows_s = O.dynamic_quant(x)
    got = O.moe_expert_quant_forward(rows_q, lay.w1_t, lay.w2_t, lay.s13, lay.s2, counts, rows_s, w2_scale_bf16=bf16_scale)
    assert got.dtype == torch.bfloat16 and got.shape == (M, 512)
    s2_used = lay.s2.to(torch.bfloat16).float() if bf16_scale else lay.s2
    s2_other = lay.s2 if bf16_scale else lay.s2.to(torch.bfloat16).float()
    wit, _ = _fp64_expert_rows(rows_q, rows_s, lay.w1_t, lay.s13, lay.w2_t, s2_used, counts)
    assert rel_err(got.float(), wit) < 6e-3 and cosine(got.float(), wit) > 0.9999
    # (b) stage 2 from the oracle's stage-1 output (both stage functions have pins of their own)
    acc1 = O.grouped_matmul_int32(rows_q, lay.w1_t, counts)
    hq, hs = O.dequant_swiglu_quant(acc1, lay.s13, rows_s, counts)
    grp = torch.repeat_interleave(torch.arange(5), counts)
    exact2 = torch.stack([hq[m].double() @ lay.w2_t[grp[m]].double() for m in range(M)])
    want = (exact2 * s2_used.double()[grp] * hs.double().unsqueeze(1)).to(torch.bfloat16)
    other = (exact2 * s2_other.double()[grp] * hs.double().unsqueeze(1)).to(torch.bfloat16)
    steps = _bf16_steps(got, want)
    assert int(steps.max()) <= 1 and float((steps == 0).float().mean()) > 0.99
    assert float((_bf16_steps(got, other) == 0).float().mean()) < 0.9, "the other scale precision is not distinguishable"
    # (c) shifted group boundaries give another result
    shifted = torch.tensor([10, 0, 22, 1, 14])
    wit_shift, _ = _fp64_expert_rows(rows_q, rows_s, lay.w1_t, lay.s13, lay.w2_t, s2_used, shifted)
    assert rel_err(got.float(), wit_shift) > 0.05


def _fp64_shared(x, w_gate_up, s_gate_up, w_down, s_down):
    """The shared expert on the W8A8 scheme in float64 (quantisation steps included)."""
    xf = x.double()
    s = xf.abs().amax(1) / 127.0
    q = torch.round(xf / s.unsqueeze(1)).clamp(-128, 127)
    d = (q @ w_gate_up.double()) * s_gate_up.double() * s.unsqueeze(1)
    inter = d.shape[1] // 2
    y = d[:, :inter] / (1 + torch.exp(-d[:, :inter])) * d[:, inter:]
    s2 = y.abs().amax(1) / 127.0
    q2 = torch.round(y / s2.unsqueeze(1)).clamp(-128, 127)
    return (q2 @ w_down.double()) * s_down.double() * s2.unsqueeze(1)


def test_deepseek_moe_forward_against_fp64_witness():
    """DeepseekMoE._forward_*_norm without collectives (deepseek_moe.py:243-368).
    (a) whole block against a permutation-free fp64 witness: library router (transformers) for the
    selection, dense brute force for the routed experts, fp64 shared expert;  a wrong expert range or a
    missing shared expert fails;  (b) the shared output is added as a bf16 tensor to the bf16 routed
    output (deepseek_moe.py:303,366), not in fp32 before the rounding: the block with the shared expert
    must equal bf16(block without + shared) bit for bit."""
    E, n_local, K, ng, tg, H, I, T = 32, 4, 8, 8, 4, 512, 256, 96
    lay = Layer(n_local, H, I, seed=33, shared=True)
    g = gen(34)
    x = tokens(T, H, 34)
    logits = torch.randn(T, E, generator=g) * 2
    logits[:, 8:12] += 2.0                      # make the local experts (ids 8..11) popular
    bias = torch.randn(E, generator=g) * 0.01
    lo = 8
    routed = (lay.w1_t, lay.s13, lay.w2_t, lay.s2)
    out, st = O.deepseek_moe_forward(x, logits, bias, routed, lay.shared, K, ng, tg, 2.5, (lo, lo + n_local),
                                     return_stages=True)
    assert out.dtype == torch.bfloat16
    # (a) independent selection and weights from the library router
    with torch.no_grad():
        _, hw, hi = _hf_router(E, K, ng, tg, 2.5, bias)(logits)
    xq, xs = O.dynamic_quant(x)
    dense_routed = O.dense_bruteforce(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, hw, hi.int(), (lo, lo + n_local))
    assert int(((hi >= lo) & (hi < lo + n_local)).sum()) > T     # the local range really is exercised
    wit = dense_routed + _fp64_shared(x, *lay.shared)
    assert rel_err(out.float(), wit) < 6e-3 and cosine(out.float(), wit) > 0.9999
    wrong_range = O.dense_bruteforce(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, hw, hi.int(), (lo + 1, lo + 1 + n_local))
    assert rel_err(out.float(), wrong_range + _fp64_shared(x, *lay.shared)) > 0.05
    assert rel_err(out.float(), dense_routed) > 0.05               # the shared expert is in the sum
    # (b) rounding points of the final add
    out_wo = O.deepseek_moe_forward(x, logits, bias, routed, None, K, ng, tg, 2.5, (lo, lo + n_local))
    sh = O.shared_expert_mlp(x, *lay.shared)
    assert out_wo.dtype == torch.bfloat16 and sh.dtype == torch.bfloat16
    assert torch.equal(out, out_wo + sh)
    fp32_add = (st["out32"] + _fp64_shared(x, *lay.shared).float()).to(torch.bfloat16)
    assert not torch.equal(out, fp32_add)                          # and that is a different number


# ------------------------------------------------------------------ gate projection with a stated order
def _fma_exact(a: float, b: float, c: float) -> float:
    """a*b + c in exact rational arithmetic, rounded once to fp32 (round to nearest even)."""
    from fractions import Fraction
    v = Fraction(a) * Fraction(b) + Fraction(c)
    if v == 0:
        return 0.0
    f = np.float32(float(v))                     # a first guess; fix it with exact comparisons
    cands = sorted({float(np.nextafter(f, np.float32(-np.inf))), float(f), float(np.nextafter(f, np.float32(np.inf)))})
    best = min(cands, key=lambda t: (abs(Fraction(t) - v), int(np.float32(t).view(np.uint32)) & 1))
    return best


def test_fma32_is_a_single_rounding():
    g = gen(40)
    a = torch.randn(4000, generator=g) * 3
    b = torch.randn(4000, generator=g) * 0.05
    c = torch.randn(4000, generator=g) * torch.logspace(-6, 6, 4000)
    # constructed double-rounding traps: c has an odd last mantissa bit, a*b is half an ulp of c minus (or
    # plus) something far below the fp64 resolution at c, so the fp64 sum is exactly the half-way point and a
    # second rounding would go to the even neighbour whatever side the exact sum is on
    traps_a, traps_b, traps_c = [], [], []
    eps = 2.0 ** -23
    for e in (10, 20, 30):
        for sa, sb in ((1, -1), (1, 1), (-1, -1)):
            for csign in (1.0, -1.0):
                c_val = csign * (2.0 ** e) * (1 + eps)                 # odd mantissa
                half_ulp = 2.0 ** (e - 24)
                root = 2.0 ** ((e - 24) / 2) if (e - 24) % 2 == 0 else None
                if root is None:
                    continue
                traps_a.append(csign * root * (1 + sa * eps))
                traps_b.append(root * (1 + sb * eps))                  # a*b = +-half_ulp * (1 +- 2^-22.. or -2^-46)
                traps_c.append(c_val)
    a = torch.cat([a, torch.tensor(traps_a)]).float()
    b = torch.cat([b, torch.tensor(traps_b)]).float()
    c = torch.cat([c, torch.tensor(traps_c)]).float()
    got = O.fma32(a, b, c)
    want = torch.tensor([_fma_exact(float(x), float(y), float(z)) for x, y, z in zip(a, b, c)], dtype=torch.float32)
    assert torch.equal(got, want)
    naive = (a.double() * b.double() + c.double()).float()
    assert not torch.equal(naive, want), "the traps do not trap: fp64 then fp32 rounding agreed everywhere"
    two_roundings = a * b + c
    assert not torch.equal(two_roundings, want)


def test_gate_logits_spec_against_fp64_matmul():
    g = gen(41)
    T, H, E = 9, 1024, 40
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    w = torch.randn(E, H, generator=g) * 0.02
    got = O.gate_logits_spec(x, w)
    ref = x.double() @ w.double().t()
    assert got.shape == (T, E) and got.dtype == torch.float32
    assert float((got.double() - ref).abs().max()) < 2e-6 * float(ref.abs().max()) + 1e-6
    # mistakes this must catch: a transposed operand, a dropped slice, a dropped last element
    assert rel_err(got, x.double() @ w.double().flip(1).t()) > 0.5
    assert float((got.double() - x.double()[:, 128:] @ w.double()[:, 128:].t()).abs().max()) > 1e-3
    assert float((got.double() - x.double()[:, :-1] @ w.double()[:, :-1].t()).abs().max()) > 1e-5
    # the order is the stated one: chains of 128, groups of 8 slices.  A plain left-to-right fp32 sum differs
    # in the last bits, the stated tree reproduced with python floats (exact fma per step) does not
    t, e = 3, 17
    xs, ws = x[t].float().tolist(), w[e].tolist()
    slices = []
    for s0 in range(0, H, 128):
        acc = 0.0
        for k in range(s0, s0 + 128):
            acc = _fma_exact(xs[k], ws[k], acc)
        slices.append(np.float32(acc))
    tot = None
    for g0 in range(0, len(slices), 8):
        q = slices[g0]
        for v in slices[g0 + 1:g0 + 8]:
            q = np.float32(q + v)
        tot = q if tot is None else np.float32(tot + q)
    assert float(got[t, e]) == float(tot)
    # bf16 weights and the bf16-rounded output of the bf16 gate
    wb = w.to(torch.bfloat16)
    got_b = O.gate_logits_spec(x, wb, round_bf16=True)
    assert torch.equal(got_b, got_b.to(torch.bfloat16).float())
    assert float((got_b.double() - x.double() @ wb.double().t()).abs().max()) < 0.01 * float(ref.abs().max())


def test_grouped_matmul_finalize_routing_closed_form():
    """``grouped_matmul_finalize_routing`` (npu_grouped_matmul_finalize_routing, fused_moe.py:536) against an fp64
    closed form that shares nothing with it: out[t] = shared[t - offset] + sum over the rows m with
    row_index[m] == t of logit[m] * (a[m] . W[g(m)]) * w_scale[g(m)] * s[m], written with a Python loop over rows
    and an exact integer product.  fp32 accumulation of at most K + 1 terms stays within a few ulp of it.
    Must-fail variants: a wrong group's scale, the shared input at offset 0 instead of its offset, a missing logit.
    For ``rows_bf16=True`` the rounding point is pinned: every row is rounded to bf16 *before* it is weighted;
    rounding after the weighting gives other bits, and so does no rounding at all."""
    g = torch.Generator().manual_seed(77)
    G, Kd, H, T, off = 3, 64, 48, 12, 5
    counts = torch.tensor([7, 0, 9])
    M = int(counts.sum())
    a = torch.randint(-128, 128, (M, Kd), generator=g, dtype=torch.int8)
    w = torch.randint(-128, 128, (G, Kd, H), generator=g, dtype=torch.int8)
    w_scale = torch.rand(G, H, generator=g) * 1e-3 + 1e-4
    s = torch.rand(M, generator=g) * 1e-2 + 1e-3
    logit = torch.rand(M, generator=g) + 0.1
    row_index = torch.randint(0, T, (M,), generator=g)
    shared = (torch.randn(4, H, generator=g)).to(torch.bfloat16)      # rows [off, off + 4) of the output
    got = O.grouped_matmul_finalize_routing(a, w, counts, w_scale, s, shared, logit, row_index, T, 1.0, off)
    assert got.dtype == torch.float32 and tuple(got.shape) == (T, H)

    def closed(scale_group_shift=0, shared_at=off, use_logit=True):
        out = torch.zeros(T, H, dtype=torch.float64)
        out[shared_at:shared_at + 4] += shared.double()
        grp = torch.repeat_interleave(torch.arange(G), counts)
        for m in range(M):
            gm = int(grp[m])
            acc = a[m].to(torch.int64) @ w[gm].to(torch.int64)            # exact
            v = acc.double() * w_scale[(gm + scale_group_shift) % G].double() * float(s[m])
            out[int(row_index[m])] += (float(logit[m]) if use_logit else 1.0) * v
        return out
    want = closed()
    tol = 8 * torch.finfo(torch.float32).eps * want.abs().clamp(min=1e-30) + 1e-12
    assert bool(((got.double() - want).abs() <= tol + 4e-7 * want.abs().max()).all())
    rel = lambda x: float((got.double() - x).norm() / x.norm())
    assert rel(want) < 1e-6
    assert rel(closed(scale_group_shift=1)) > 1e-2          # a row dequantised with another group's scale
    assert rel(closed(shared_at=0)) > 1e-2                  # the shared rows at offset 0 instead of `off`
    assert rel(closed(use_logit=False)) > 1e-2              # the routing weight dropped
    # rows outside [off, off + 4) start from zero, rows inside from the shared input: exact on a row nobody routes to
    free = [t for t in range(T) if not bool((row_index == t).any())]
    for t in free:
        exp = shared[t - off].float() if off <= t < off + 4 else torch.zeros(H)
        assert torch.equal(got[t], exp)

    # ---- rows_bf16: rounding before the weight
    got_bf = O.grouped_matmul_finalize_routing(a, w, counts, w_scale, s, shared, logit, row_index, T, 1.0, off,
                                               rows_bf16=True)
    acc = O.grouped_matmul_int32(a, w, counts)
    grp = torch.repeat_interleave(torch.arange(G), counts)
    deq = (acc.float() * w_scale[grp]) * s.unsqueeze(-1)                 # the operator's dequantisation (C8)

    def combine(rows_fp32):
        out = torch.zeros(T, H)
        out[off:off + 4] = shared.float()
        for m in range(M):                                               # ascending m, fp32, as the oracle states
            out[int(row_index[m])] += rows_fp32[m]
        return out
    before = combine(logit.unsqueeze(-1) * deq.to(torch.bfloat16).float())
    after = combine((logit.unsqueeze(-1) * deq).to(torch.bfloat16).float())
    assert torch.equal(got_bf, before)
    assert not torch.equal(got_bf, after) and not torch.equal(got_bf, got)
    # and each rounded row is within half a bf16 step of the fp32 row it came from
    assert bool(((deq.to(torch.bfloat16).float() - deq).abs() <= deq.abs() * 2.0 ** -8).all())


def _a2_bruteforce(xq, xs, w1, w2, s1, s2, topk_w, topk_ids, expert_range, smooth, where="before"):
    """fp64, permutation free, one expert at a time on the whole batch.  `where` places the smoothing factors:
    "before" the row quantisation (the operator's order: quant_scale of npu_dequant_swiglu_quant), "none", or
    "after" (on the quantised values instead) -- the last two are the mistakes the pin has to tell apart."""
    lo, hi = expert_range
    out = torch.zeros(xq.shape[0], w2.shape[2], dtype=torch.float64)
    for e in range(lo, hi):
        sel = topk_ids == e
        tok = sel.any(dim=1)
        if not bool(tok.any()):
            continue
        wt = (topk_w.double() * sel).sum(dim=1)[tok]
        acc = xq[tok].to(torch.int64) @ w1[e - lo].to(torch.int64)
        d = acc.double() * s1[e - lo].double() * xs[tok].double().unsqueeze(-1)
        inter = d.shape[1] // 2
        y = d[:, :inter] / (1.0 + torch.exp(-d[:, :inter])) * d[:, inter:]
        if where == "before":
            y = y * smooth[e - lo].double()
        sc = y.abs().amax(dim=1) / 127.0
        q = torch.round(y / sc.clamp(min=1e-300).unsqueeze(-1)).clamp(-128, 127)
        if where == "after":
            q = q * smooth[e - lo].double()
        out[tok] += wt.unsqueeze(-1) * ((q @ w2[e - lo].double()) * s2[e - lo].double() * sc.unsqueeze(-1))
    return out


def test_a2_pipeline_against_bruteforce():
    """``fused_experts_w8a8_allgather_ep_a2`` (fused_moe.py:844-937): with smoothing factors of one it is the A3
    pipeline bit for bit (the reference's ``smooth_scale`` is ``torch.ones``, compressed_tensors_moe.py:113);
    with other factors it follows the brute force that smooths before the row quantisation and not the ones that
    drop the factors or apply them to the quantised values; the ``pd_seperate_prefill`` tail (bf16 rows, bf16
    routing weights, bf16 w2 scale) stays within the bf16 bar of the same brute force and differs from the fp32
    tail; an assignment outside the rank's range contributes nothing in either tail."""
    T, K, n_local, E, H, I = 48, 4, 4, 16, 256, 128
    lay = Layer(n_local, H, I, seed=31)
    g = gen(32)
    x = tokens(T, H, 33)
    xq, xs = O.dynamic_quant(x)
    ids = torch.rand(T, E, generator=g).argsort(1)[:, :K].int()
    w = torch.rand(T, K, generator=g)
    rng = (4, 4 + n_local)
    ones = torch.ones(n_local, I)
    a3 = O.fused_experts_w8a8_allgather_ep(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, rng)
    a2 = O.fused_experts_w8a8_allgather_ep_a2(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, rng, ones)
    assert torch.equal(a2, a3)
    smooth = torch.rand(n_local, I, generator=g) * 1.5 + 0.25
    got = O.fused_experts_w8a8_allgather_ep_a2(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, rng, smooth).double()
    brute = {k: _a2_bruteforce(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, rng, smooth, k)
             for k in ("before", "none", "after")}
    assert rel_err(got, brute["before"]) < 5e-3
    assert rel_err(got, brute["none"]) > 5e-2
    # smoothing the quantised values differs from the operator's order by the quantisation noise only: small, but
    # several times what separates the oracle from the brute force that has the order right
    assert rel_err(got, brute["after"]) > 1e-2 > 2 * rel_err(got, brute["before"])
    # tokens without a local expert get exactly zero
    none_local = ~((ids >= rng[0]) & (ids < rng[1])).any(dim=1)
    assert bool(none_local.any()) and bool((got[none_local] == 0).all())
    # the bf16 tail
    pd = O.fused_experts_w8a8_allgather_ep_a2(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, rng, smooth,
                                              pd_seperate_prefill=True)
    assert pd.dtype == torch.bfloat16 and rel_err(pd.double(), brute["before"]) < 1e-2
    assert not torch.equal(pd.float(), got.float()) and bool((pd[none_local] == 0).all())
    # its rounding points: rows to bf16 with a bf16 w2 scale, weights to bf16, fp32 sum in ascending k
    _, st = O.fused_experts_w8a8_allgather_ep_a2(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, rng, smooth,
                                                 pd_seperate_prefill=True, return_stages=True)
    counts, idx = st["counts"], st["idx"].long()
    acc2 = O.grouped_matmul_int32(st["h_q"], lay.w2_t, counts)
    grp = torch.repeat_interleave(torch.arange(n_local), counts)
    rows = ((acc2.float() * lay.s2.to(torch.bfloat16).float()[grp]) * st["h_s"].unsqueeze(-1)).to(torch.bfloat16)
    slot_of = {int(s): m for m, s in enumerate(idx)}
    want = torch.zeros(T, H)
    wb = w.to(torch.bfloat16).float()
    for n in range(T):
        for k in range(K):
            m = slot_of.get(n * K + k)
            if m is not None:
                want[n] += wb[n, k] * rows[m].float()
    assert torch.equal(pd, want.to(torch.bfloat16))
