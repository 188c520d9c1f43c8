#!/usr/bin/env python3
"""Benchmark of the W8A8 fused-MoE layer on one MI355X.

A step is one pass of the layer over one batch of synthetic tokens, inputs resident in HBM:
    router (sigmoid + bias, 8 groups / top-4, top-8)  ->  per-token int8 quantisation  ->
    sort by expert  ->  int8 GEMM1 + dequant + SwiGLU + requant  ->  int8 GEMM2 + dequant  ->
    weighted combine + shared expert.
Workloads (BASELINE.json configs):
    decode   DeepSeek-V3 shape, 32 local experts of 256 + 1 shared expert, 64 tokens
    prefill  same layer, 8192 tokens with 0.1 % outlier channels x50
Router logits are random over the 32 local experts and -30 elsewhere, so the router itself
sends every token to 8 distinct local experts ("uniform random routing into local experts").
The gate GEMM that makes the logits is not part of the step; `block_us` times the whole block
(gate included) through DeepseekMoE.forward.

The default run measures both halves of the metric and prints one JSON line: the headline is the
decode layer time with the roofline figure of its dominant kernel (GEMM1) and the CPU oracle timed on
this box's host cores; the `prefill` object carries the 8192-token layer time, its share of the int8
peak, the rooflines of both tile GEMM kernels and the deviation from the oracle.  `--workload decode`
or `--workload prefill` runs one half only (profiling runs).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12       # B/s, MI355X published
INT8_PEAK = 5.0e15      # op/s, MI355X published dense int8 (256 CU x 8192 op/clk x 2.4 GHz = 5.03e15)

# HBM-side bytes per launch of the GEMM1 kernels as recorded from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs
# of this file (scaled by what the same counters read for the 1 GiB copies of --copy-probe).  Counters cannot
# be read from inside a timed run, so these are values of record, labelled with the summary they come from.
RECORDED_TRAFFIC = {
    ("decode", "gemm1"): (996_346_000, "profiles/decode_gemm1_hbm_traffic.txt"),
    ("prefill", "gemm1"): (5437806000, "profiles/prefill_gemm1_hbm_traffic.txt"),
    ("prefill", "gemm2"): (5072506000, "profiles/prefill_gemm1_hbm_traffic.txt"),
}

SHAPES = {
    "decode": dict(T=64, H=7168, I=2048, E=256, n_local=32, K=8, n_group=8, topk_group=4, scale=2.5, outlier=0.0),
    "prefill": dict(T=8192, H=7168, I=2048, E=256, n_local=32, K=8, n_group=8, topk_group=4, scale=2.5,
                    outlier=0.001),
}


def make_weights(n_local, H, I, seed, dev):
    """fp32 N(0, 0.02) weights quantised to symmetric per-output-channel int8 (checkpoint layout)."""
    g = torch.Generator(device=dev).manual_seed(seed)

    def q(out_f, in_f):
        w = torch.randn(out_f, in_f, generator=g, device=dev) * 0.02
        s = w.abs().amax(dim=1) / 127.0
        return torch.round(w / s.unsqueeze(1)).clamp(-127, 127).to(torch.int8), s

    w13 = torch.empty(n_local, 2 * I, H, dtype=torch.int8, device=dev)
    w2 = torch.empty(n_local, H, I, dtype=torch.int8, device=dev)
    s13 = torch.empty(n_local, 2 * I, device=dev)
    s2 = torch.empty(n_local, H, device=dev)
    for e in range(n_local):
        w13[e], s13[e] = q(2 * I, H)
        w2[e], s2[e] = q(H, I)
    return w13, s13, w2, s2


class WeightSet:
    def __init__(self, cfg, seed, dev):
        from omni_infer_amd import hip_ops as ops
        H, I, n = cfg["H"], cfg["I"], cfg["n_local"]
        w13, self.s13, w2, self.s2 = make_weights(n, H, I, seed, dev)
        sw13, ss13, sw2, ss2 = make_weights(1, H, I, seed + 1000, dev)
        self.ckpt = (w13, w2, sw13[0], sw2[0])          # kept for the CPU baseline (set 0 only)
        self.w13 = ops.pack_weight(w13, 1)
        self.w2 = ops.pack_weight(w2, 1)
        self.sh13 = ops.pack_weight(sw13[0], 1)
        self.sh2 = ops.pack_weight(sw2[0], 1)
        self.sh_s13, self.sh_s2 = ss13[0].contiguous(), ss2[0].contiguous()

    def drop_ckpt(self):
        self.ckpt = None


def make_inputs(cfg, dev):
    g = torch.Generator().manual_seed(0)
    T, H, E, n_local = cfg["T"], cfg["H"], cfg["E"], cfg["n_local"]
    x = torch.randn(T, H, generator=g)
    if cfg["outlier"] > 0:
        n = max(1, int(round(H * cfg["outlier"])))
        ch = torch.randperm(H, generator=g)[:n]
        x[:, ch] *= 50.0
    if cfg.get("routing") == "global_filter":
        # every expert of the model can be chosen: what a rank sees after the all-gather of the tokens, of which
        # it keeps the assignments to its own experts (about T rows)
        logits = torch.randn(T, E, generator=g)
    else:
        # local_dense: every token's K experts are local ones (what a rank receives after a dispatch: K * T rows)
        logits = torch.full((T, E), -30.0)
        logits[:, :n_local] = torch.randn(T, n_local, generator=g)
    bias = torch.randn(E, generator=g) * 0.01
    return x.to(torch.bfloat16).to(dev), logits.to(dev), bias.to(dev)


def noaux_tc_routing(cfg):
    """The routing arguments of npu_moe_gating_top_k as the reference calls it (layer.py:341-351): sigmoid scores,
    bias for the selection only, groups ranked by the sum of their two best, weights renormalised and scaled."""
    from omni_infer_amd import _lib as L
    return dict(top_k=cfg["K"], n_group=cfg["n_group"], topk_group=cfg["topk_group"], score_fn="sigmoid",
                group_mode=L.OMNI_GROUP_TOP2SUM, masked_fill_zero=False, weight_from_c=False, renorm=True,
                scale=cfg["scale"], eps=1e-20)


def algorithmic_bytes_layer(cfg, groups_active):
    H, I, T = cfg["H"], cfg["I"], cfg["T"]
    w = groups_active * (H * 2 * I + I * H)
    sc = groups_active * (2 * I + H) * 4
    return w + sc + T * H * 2 + T * H * 2


def algorithmic_ops_layer(cfg, rows_routed):
    H, I, T = cfg["H"], cfg["I"], cfg["T"]
    return 2 * (rows_routed + T) * (H * 2 * I + I * H)


def cpu_baseline(cfg, ws, x, logits, bias, sample_tokens, rows_bf16=False):
    """The oracle's whole layer on the host cores, on the first `sample_tokens` tokens."""
    from oracle import moe_oracle as O
    torch.set_num_threads(os.cpu_count() or 1)
    w13, w2, sw13, sw2 = [t.cpu() for t in ws.ckpt]
    routed = (w13.transpose(1, 2).contiguous(), ws.s13.cpu(), w2.transpose(1, 2).contiguous(), ws.s2.cpu())
    shared = (sw13.t().contiguous(), ws.sh_s13.cpu(), sw2.t().contiguous(), ws.sh_s2.cpu())
    xs, ls, b = x[:sample_tokens].cpu(), logits[:sample_tokens].cpu(), bias.cpu()

    def run():
        if rows_bf16:   # the library's bf16-row option: the same block with every expert row rounded before the sum
            w, ids = O.route_noaux_tc(ls, b, cfg["K"], cfg["n_group"], cfg["topk_group"], cfg["scale"])
            xq, xsc = O.dynamic_quant(xs)
            o = O.fused_experts_w8a8_allgather_ep(xq, xsc, routed[0], routed[2], routed[1], routed[3], w, ids,
                                                  (0, cfg["n_local"]), rows_bf16=True)
            return o + O.shared_expert_mlp(xs, *shared)
        return O.deepseek_moe_forward(xs, ls, b, routed, shared, cfg["K"], cfg["n_group"], cfg["topk_group"],
                                      cfg["scale"], (0, cfg["n_local"]))
    out = run()  # untimed first pass (thread pool, page faults)
    # about ten seconds of host work, whole passes only
    reps, t0 = 0, time.perf_counter()
    while reps < 3 or (time.perf_counter() - t0 < 10.0 and reps < 1000):
        out = run()
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    return dt, reps, out


def bench_norm(args):
    """Secondary workload: the producer in front of the block (residual add + RMSNorm + dynamic quant,
    all three outputs) on 8192 x 7168 bf16 rows.  One step = one launch; input sets are rotated so that
    the rows come from HBM."""
    from omni_infer_amd import _lib as L
    from omni_infer_amd import hip_ops as ops
    T, H, eps = 8192, 7168, 1e-6
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(0)
    nsets = 4
    xs = [torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16) for _ in range(nsets)]
    rs = [torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16) for _ in range(nsets)]
    w = (1.0 + 0.1 * torch.randn(H, generator=g, device=dev)).to(torch.bfloat16)
    y = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    ro = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    q = torch.empty(T, H, dtype=torch.int8, device=dev)
    sc = torch.empty(T, dtype=torch.float32, device=dev)
    lib, st = L.lib(), torch.cuda.current_stream().cuda_stream

    def step(i):
        rc = lib.omni_add_rms_norm_quant(xs[i % nsets].data_ptr(), rs[i % nsets].data_ptr(), w.data_ptr(), T, H, eps,
                                         ro.data_ptr(), y.data_ptr(), q.data_ptr(), sc.data_ptr(), st)
        L.check(rc, "omni_add_rms_norm_quant")
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(args.steps):
        step(i)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / args.steps
    alg = T * H * (2 + 2 + 2 + 2 + 1) + T * 4 + H * 2     # x, residual in; residual, y, int8 out; scales; weight
    result = {"metric": "add_rms_norm_quant_latency", "value": ms * 1e3, "unit": "us", "n_gpus": 1, "steps": args.steps,
              "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": False, "scaling": "weak",
              "vs_baseline": None, "dtype": "f32", "data": "synthetic",
              "config": {"workload": f"residual add + RMSNorm + per-token int8 quantisation, {T} x {H} bf16 rows, "
                                     "outputs: residual, normalised rows, int8 rows + scales", "rows": T, "H": H},
              "roofline": {"bound": "hbm", "kernel": "add_rms_norm_quant_kernel", "achieved": alg / (ms * 1e-3) / 1e9,
                           "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": alg / (ms * 1e-3) / HBM_PEAK,
                           "kernel_us": ms * 1e3, "algorithmic_per_launch": alg, "traffic": None}}
    if not args.no_cpu:
        from oracle import moe_oracle as O
        torch.set_num_threads(os.cpu_count() or 1)
        n = 1024
        xc, rc_, wc = xs[0][:n].cpu(), rs[0][:n].cpu(), w.cpu()
        O.add_rms_norm_dynamic_quant(xc, rc_, wc, eps)
        t0 = time.perf_counter()
        for _ in range(3):
            qr, sr, rr = O.add_rms_norm_dynamic_quant(xc, rc_, wc, eps)
        dt = (time.perf_counter() - t0) / 3
        step(0)
        torch.cuda.synchronize()
        result["cpu_baseline"] = {"value": dt * 1e6 * (T / n), "unit": "us", "cores": torch.get_num_threads(),
                                  "kind": "port", "sample": f"oracle on the first {n} of {T} rows, scaled by rows",
                                  "gpu_vs_oracle_bit_exact": bool(torch.equal(q[:n].cpu(), qr) and
                                                                  torch.equal(sc[:n].cpu(), sr) and
                                                                  torch.equal(ro[:n].cpu(), rr))}
    print(json.dumps(result))


PREHEAT_S = 0.3   # untimed, reported: the same step repeated for this long before the warm-up steps


def preheat(fn, seconds=PREHEAT_S, max_steps=20000):
    """Runs fn(i) untimed for about `seconds` of GPU time and returns the number of calls made.  A run of a few
    dozen steps is over before the chip has left its idle clocks; with this in front, a short timed region
    reads what a long one reads (the steady state of a serving loop)."""
    n, t0 = 0, time.perf_counter()
    while n < max_steps and time.perf_counter() - t0 < seconds:
        for _ in range(16):
            fn(n)
            n += 1
        torch.cuda.synchronize()
    return n


def time_steps(fn, steps, warmup, preheat_s=0.0):
    """Average GPU time of `steps` calls of fn(i) after `warmup` untimed ones (events on torch's current
    stream, which is the stream every library call is enqueued on), plus the host wall time per step."""
    time_steps.last_preheat = preheat(fn, preheat_s) if preheat_s > 0 else 0
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        fn(i)
    e1.record()
    torch.cuda.synchronize()
    return max(e0.elapsed_time(e1) / steps, 0.0), (time.perf_counter() - t0) * 1e3 / steps


def single_step_spread(fn, n):
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for i, (a0, a1) in enumerate(evs):
        a0.record()
        fn(i)
        a1.record()
    torch.cuda.synchronize()
    per = sorted(a0.elapsed_time(a1) * 1e3 for a0, a1 in evs)
    return {"p10": per[int(0.1 * (n - 1))], "p50": per[(n - 1) // 2], "p90": per[int(0.9 * (n - 1))]}


def graph_replay_us(step, n_sets, steps):
    """The same steps replayed from a HIP graph (how a serving stack runs the decode path): one graph holds one
    step per weight set, so the rotation of the eager loop is kept; average time of a step over the replays.
    The capture runs on a stream of its own; the library calls record kernel launches only (no memset nodes)."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        for i in range(n_sets):
            step(i)                       # per-device look-ups of the library happen outside the capture
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for i in range(n_sets):
                step(i)
    torch.cuda.current_stream().wait_stream(side)
    replays = max(1, steps // n_sets)
    preheat(lambda i: graph.replay(), PREHEAT_S / 3)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(replays):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / (replays * n_sets)


def measure_layer(name, sets, steps, warmup, rows_dtype, no_cpu, dev, kernel_steps=None):
    """One workload: whole-layer time, both GEMM kernels alone, the byte / op counts of the routing that
    the router produced, and (unless no_cpu) the oracle on a bounded sample of the same tokens."""
    from omni_infer_amd import _lib as L
    from omni_infer_amd import hip_ops as ops
    cfg = SHAPES[name]
    T, H, I, K, n_local = cfg["T"], cfg["H"], cfg["I"], cfg["K"], cfg["n_local"]
    x, logits, bias = make_inputs(cfg, dev)
    need = L.lib().omni_moe_w8a8_layer_workspace_bytes(T, K, n_local, H, I, 1, ops._DT[rows_dtype])
    workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)

    topk_w = torch.empty(T, K, dtype=torch.float32, device=dev)
    topk_ids = torch.empty(T, K, dtype=torch.int32, device=dev)

    def step(i):
        # router (npu_moe_gating_top_k as called at layer.py:341-351) and layer in one library call
        ws = sets[i % len(sets)]
        return ops.moe_w8a8_layer_routed(x, None, logits, bias, lo=0, hi=n_local, w13_packed=ws.w13, w13_scale=ws.s13,
                                         w2_packed=ws.w2, w2_scale=ws.s2,
                                         shared=(ws.sh13, ws.sh_s13, ws.sh2, ws.sh_s2), H=H, I=I, workspace=workspace,
                                         out=out, rows_dtype=rows_dtype, topk_w=topk_w, topk_ids=topk_ids,
                                         **noaux_tc_routing(cfg))[0]

    ms, wall_ms = time_steps(step, steps, warmup, PREHEAT_S)
    preheat_steps = time_steps.last_preheat
    spread = single_step_spread(step, min(50, steps))
    graph_us = None
    if name == "decode":
        try:
            graph_us = graph_replay_us(step, len(sets), steps)
        except RuntimeError as e:      # a capture the runtime refuses must not cost the line its other figures
            print(f"bench.py: graph replay not measured: {e}", file=sys.stderr)

    # routing actually produced (rows per local expert) for the byte / op counts
    w, ids, _ = ops.npu_moe_gating_top_k(logits, K, bias, cfg["topk_group"], cfg["n_group"], 1, 0, 1, cfg["scale"], 1e-20)
    p = ops.moe_permute(ids, 0, n_local, L.OMNI_IDX_TOKEN_MAJOR)
    counts = p.counts.cpu()
    rows_routed = int(counts.sum())
    active = int((counts > 0).sum()) + 1
    rows_total = rows_routed + T
    layer_bytes = algorithmic_bytes_layer(cfg, active)
    layer_ops = algorithmic_ops_layer(cfg, rows_routed)

    # ---- the two GEMM kernels alone, each timed with events on its stream.  GEMM1 is called with
    # OMNI_GEMM1_NO_REQUANT, which stops after the GEMM kernel, and OMNI_GEMM1_WS_ZEROED (the workspace below is
    # zero-filled once), so that the streaming kernel runs as it does inside the layer, without a launch that clears
    # its counters; the tile kernel is preceded by the one-block fill kernel that clears its split-tile counters
    # (about 2 us, inside the figure)
    M_cap = T * K + T
    xq, xs = ops.npu_dynamic_quant(x)
    g1_ws = torch.zeros(L.lib().omni_moe_gemm1_workspace_bytes(T, K, n_local, T, M_cap, H, I), dtype=torch.uint8, device=dev)
    hq = torch.empty(M_cap, I, dtype=torch.int8, device=dev)
    hs = torch.empty(M_cap, dtype=torch.float32, device=dev)
    rows = torch.empty(M_cap, H, dtype=rows_dtype, device=dev)

    def gemm1_only(i):
        ws = sets[i % len(sets)]
        ops.grouped_gemm1_swiglu_quant(xq, xs, p.sorted_src, L.OMNI_IDX_TOKEN_MAJOR, K, ws.w13, ws.s13, p.offsets, H, I,
                                       M_cap, extra=(ws.sh13, ws.sh_s13), extra_rows=T,
                                       flags=L.OMNI_GEMM1_NO_REQUANT | L.OMNI_GEMM1_WS_ZEROED, workspace=g1_ws, out=(hq, hs))

    def gemm2_only(i):
        ws = sets[i % len(sets)]
        ops.grouped_gemm2_dequant(hq, hs, ws.w2, ws.s2, p.offsets, H, I, out_dtype=rows_dtype,
                                  extra=(ws.sh2, ws.sh_s2), extra_rows=T, out=rows, workspace=g1_ws)

    ops.grouped_gemm1_swiglu_quant(xq, xs, p.sorted_src, L.OMNI_IDX_TOKEN_MAJOR, K, sets[0].w13, sets[0].s13, p.offsets,
                                   H, I, M_cap, extra=(sets[0].sh13, sets[0].sh_s13), extra_rows=T, workspace=g1_ws,
                                   out=(hq, hs))                       # real int8 rows for GEMM2 to read
    ksteps = kernel_steps or max(10, steps // 2)
    k1_ms, _ = time_steps(gemm1_only, ksteps, 5, PREHEAT_S / 3)
    k2_ms, _ = time_steps(gemm2_only, ksteps, 5, PREHEAT_S / 3)
    name1 = ops.gemm_kernel_name(1, T, K, n_local, T, M_cap, H, I)
    name2 = ops.gemm_kernel_name(2, T, K, n_local, T, M_cap, H, I)
    rows_bytes = 4 if rows_dtype == torch.float32 else 2
    if name == "decode":
        # weights and scales of every active group + the int8 tokens (intermediates are implementation traffic)
        alg1 = active * (H * 2 * I + 2 * I * 4) + T * H
        alg2 = active * (I * H + H * 4) + rows_total * I
        roofs = [dict(bound="hbm", kernel=name1, achieved=alg1 / (k1_ms * 1e-3) / 1e9, peak=HBM_PEAK / 1e9, unit="GB/s",
                      kernel_us=k1_ms * 1e3, algorithmic_per_launch=alg1),
                 dict(bound="hbm", kernel=name2, achieved=alg2 / (k2_ms * 1e-3) / 1e9, peak=HBM_PEAK / 1e9, unit="GB/s",
                      kernel_us=k2_ms * 1e3, algorithmic_per_launch=alg2)]
    else:
        alg1 = 2 * rows_total * H * 2 * I
        alg2 = 2 * rows_total * I * H
        roofs = [dict(bound="mfma", kernel=name1, achieved=alg1 / (k1_ms * 1e-3) / 1e12, peak=INT8_PEAK / 1e12,
                      unit="TFLOP/s", kernel_us=k1_ms * 1e3, algorithmic_per_launch=alg1),
                 dict(bound="mfma", kernel=name2, achieved=alg2 / (k2_ms * 1e-3) / 1e12, peak=INT8_PEAK / 1e12,
                      unit="TFLOP/s", kernel_us=k2_ms * 1e3, algorithmic_per_launch=alg2)]
    for r, key in zip(roofs, ("gemm1", "gemm2")):
        r["frac"] = r["achieved"] / r["peak"]
        rec = RECORDED_TRAFFIC.get((name, key))
        r["traffic"] = rec[0] if rec else None
        if rec:
            r["traffic_source"] = rec[1]
    res = {
        "workload": f"DeepSeek-V3-shape W8A8 MoE layer, {name}: {T} tokens, {n_local} local experts of {cfg['E']} + 1 shared, "
                    f"H={H}, I={I}, top-{K} grouped sigmoid routing",
        "tokens": T, "rows_routed": rows_routed, "active_groups": active, "rows_dtype": str(rows_dtype).split(".")[-1],
        "layer_us": ms * 1e3, "ms_per_step": ms, "steps": steps, "warmup": warmup, "preheat_steps": preheat_steps,
        "graph_us": graph_us,
        "algorithmic_bytes": layer_bytes, "algorithmic_ops": layer_ops,
        "hbm_frac": layer_bytes / (ms * 1e-3) / HBM_PEAK, "int8_frac": layer_ops / (ms * 1e-3) / INT8_PEAK,
        "host_wall_ms_per_step": wall_ms, "single_step_us": spread,
        "roofline_gemm1": roofs[0], "roofline_gemm2": roofs[1],
    }
    if not no_cpu:
        sample = T if name == "decode" else 1024
        dt, reps, ref = cpu_baseline(cfg, sets[0], x, logits, bias, sample, rows_dtype == torch.bfloat16)
        got = step(0)[:sample].float().cpu()
        torch.cuda.synchronize()
        refd = ref.float()
        res["cpu_baseline"] = {"value": dt * 1e6 * (T / sample), "unit": "us", "cores": torch.get_num_threads(),
                               "kind": "port",
                               "sample": f"oracle layer on the first {sample} of {T} tokens "
                                         f"({reps} passes of {dt:.3f} s" + (", scaled by tokens)" if sample != T else ")"),
                               "gpu_vs_oracle_rel_err": float((got - refd).norm() / refd.norm()),
                               "gpu_vs_oracle_bit_exact": bool(torch.equal(got, refd))}
    return res, step


def measure_global_filter(sets, steps, warmup, rows_dtype, dev):
    """The prefill token count with the routing of the all-gather form of expert parallelism (router over all
    256 experts, the local range filter keeps about T assignments): layer time against both rooflines."""
    from omni_infer_amd import _lib as L
    from omni_infer_amd import hip_ops as ops
    cfg = dict(SHAPES["prefill"], routing="global_filter")
    T, H, I, K, n_local = cfg["T"], cfg["H"], cfg["I"], cfg["K"], cfg["n_local"]
    x, logits, bias = make_inputs(cfg, dev)
    need = L.lib().omni_moe_w8a8_layer_workspace_bytes(T, K, n_local, H, I, 1, ops._DT[rows_dtype])
    workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)

    topk_w = torch.empty(T, K, dtype=torch.float32, device=dev)
    topk_ids = torch.empty(T, K, dtype=torch.int32, device=dev)

    def step(i):
        # router (npu_moe_gating_top_k as called at layer.py:341-351) and layer in one library call
        ws = sets[i % len(sets)]
        return ops.moe_w8a8_layer_routed(x, None, logits, bias, lo=0, hi=n_local, w13_packed=ws.w13, w13_scale=ws.s13,
                                         w2_packed=ws.w2, w2_scale=ws.s2,
                                         shared=(ws.sh13, ws.sh_s13, ws.sh2, ws.sh_s2), H=H, I=I, workspace=workspace,
                                         out=out, rows_dtype=rows_dtype, topk_w=topk_w, topk_ids=topk_ids,
                                         **noaux_tc_routing(cfg))[0]

    ms, _ = time_steps(step, steps, warmup, PREHEAT_S / 3)

    def step_routed_only(i):
        # the reference runs the shared expert on the rank's own tokens before the all-gather (deepseek_moe.py:244):
        # on the gathered tokens only the routed experts are computed
        ws = sets[i % len(sets)]
        return ops.moe_w8a8_layer_routed(x, None, logits, bias, lo=0, hi=n_local, w13_packed=ws.w13, w13_scale=ws.s13,
                                         w2_packed=ws.w2, w2_scale=ws.s2, shared=None, H=H, I=I, workspace=workspace,
                                         out=out, rows_dtype=rows_dtype, topk_w=topk_w, topk_ids=topk_ids,
                                         **noaux_tc_routing(cfg))[0]

    ms_routed, _ = time_steps(step_routed_only, steps, warmup, PREHEAT_S / 3)
    w, ids, _ = ops.npu_moe_gating_top_k(logits, K, bias, cfg["topk_group"], cfg["n_group"], 1, 0, 1, cfg["scale"], 1e-20)
    counts = ops.moe_permute(ids, 0, n_local, L.OMNI_IDX_TOKEN_MAJOR).counts.cpu()
    rows_routed, active = int(counts.sum()), int((counts > 0).sum()) + 1
    M_cap = T * K + T
    return {"routing": "router over all 256 experts, assignments to the 32 local ones kept", "tokens": T,
            "rows_routed": rows_routed, "rows_of_busiest_expert": int(counts.max()), "active_groups": active,
            "rows_dtype": str(rows_dtype).split(".")[-1], "layer_us": ms * 1e3, "steps": steps,
            "routed_experts_only_us": ms_routed * 1e3,
            "routed_experts_only_hbm_frac": algorithmic_bytes_layer(cfg, active - 1) / (ms_routed * 1e-3) / HBM_PEAK,
            "routed_experts_only_int8_frac": 2 * rows_routed * (H * 2 * I + I * H) / (ms_routed * 1e-3) / INT8_PEAK,
            "gemm1_kernel": ops.gemm_kernel_name(1, T, K, n_local, T, M_cap, H, I),
            "hbm_frac": algorithmic_bytes_layer(cfg, active) / (ms * 1e-3) / HBM_PEAK,
            "int8_frac": algorithmic_ops_layer(cfg, rows_routed) / (ms * 1e-3) / INT8_PEAK}


def measure_block(name, ws, steps, warmup, dev):
    """The whole MoE block through DeepseekMoE.forward (gate GEMM, router, layer; fused body): what a model
    pays per layer call.  Weights are those of one weight set (no rotation: about the cache-resident share
    of 1.45 GB is served from the last-level cache, so this figure is a lower bound next to `value`)."""
    import types
    from omni_infer_amd import config, distributed
    from omni_infer_amd.layers.deepseek_moe import DeepseekMoE
    from omni_infer_amd.quantization.compressed_tensors import AscendCompressedTensorsConfig
    cfg = SHAPES[name]
    T, H, I, K, n_local, E = cfg["T"], cfg["H"], cfg["I"], cfg["K"], cfg["n_local"], cfg["E"]
    config.update_model_extra_config(enable_moe_expert_parallel=True, moe_dispatch_combine=False,
                                     prefill_dispatch_combine=False)
    distributed.set_virtual_ep(E // n_local, 0)
    mc = types.SimpleNamespace(hidden_size=H, n_routed_experts=E, num_experts_per_tok=K, moe_intermediate_size=I,
                               n_shared_experts=1, n_group=cfg["n_group"], topk_group=cfg["topk_group"],
                               norm_topk_prob=True, scoring_func="sigmoid", topk_method="noaux_tc",
                               routed_scaling_factor=cfg["scale"], hidden_act="silu", first_k_dense_replace=3)
    blk = DeepseekMoE(mc, AscendCompressedTensorsConfig(ignore=["gate"]), prefix="model.layers.3.mlp", device=dev)
    g = torch.Generator(device=dev).manual_seed(7)
    gate_w = torch.randn(E, H, generator=g, device=dev) * 0.02
    gate_w[n_local:] = 0.0            # the other ranks' experts score sigmoid(0) + a negative bias: never chosen
    blk.gate.weight.data.copy_(gate_w)
    bias = torch.randn(E, generator=g, device=dev) * 0.01
    bias[n_local:] -= 10.0
    blk.gate.e_score_correction_bias.data.copy_(bias)
    w13, w2, sw13, sw2 = ws.ckpt
    ex, se = blk.experts, blk.shared_experts
    ex.w13_weight.data.copy_(w13)
    ex.w2_weight.data.copy_(w2)
    ex.w13_weight_scale.data.copy_(ws.s13)
    ex.w2_weight_scale.data.copy_(ws.s2)
    se.gate_up_proj.weight.data.copy_(sw13)
    se.gate_up_proj.weight_scale.data.copy_(ws.sh_s13.unsqueeze(-1))
    se.down_proj.weight.data.copy_(sw2)
    se.down_proj.weight_scale.data.copy_(ws.sh_s2.unsqueeze(-1))
    blk.process_weights_after_loading()
    x, _, _ = make_inputs(cfg, dev)

    def step(i):
        return blk(x, None, None, 3)
    ms, wall_ms = time_steps(step, steps, warmup, PREHEAT_S / 3)
    ids = blk._route(x)[1]
    local = int(((ids >= 0) & (ids < n_local)).sum())
    return {"block_us": ms * 1e3, "host_wall_ms_per_step": wall_ms, "steps": steps, "local_assignments": local,
            "tokens": T}


def bench_calib(args):
    """What the hardware delivers on this box, to read the layer's figures against (one JSON line):
    the int8 matrix instruction alone on zero and on random operands, the vendor library's plain int8 GEMM
    (torch._int_mm) at the shapes of the two prefill GEMMs, a device-to-device copy and a kernel that only reads."""
    from omni_infer_amd import _lib as L
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    lib, st = L.lib(), torch.cuda.current_stream().cuda_stream
    props = torch.cuda.get_device_properties(dev)
    cus = props.multi_processor_count
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    res = {"metric": "hardware_calibration", "unit": "POPS", "n_gpus": 1, "data": "synthetic", "cus": cus,
           "int8_peak_published_pops": INT8_PEAK / 1e15}

    def ev_ms(fn, reps):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    iters, g = 20000, torch.Generator(device=dev).manual_seed(0)
    for name, ops_buf in (("zeros", torch.zeros(1 << 16, dtype=torch.int8, device=dev)),
                          ("random_uniform", torch.randint(-128, 128, (1 << 16,), generator=g, device=dev, dtype=torch.int8)),
                          ("gaussian_sigma30", (torch.randn(1 << 16, generator=g, device=dev) * 30).clamp(-127, 127).to(torch.int8))):
        def run():
            L.check(lib.omni_diag_mfma_i8_rate(ops_buf.data_ptr(), ops_buf.numel(), iters, cus, sink.data_ptr(), st),
                    "omni_diag_mfma_i8_rate")
        ms = ev_ms(run, 5)
        ops_total = cus * 8 * 8 * iters * 65536.0
        res[f"mfma_i8_{name}_pops"] = ops_total / (ms * 1e-3) / 1e15
        res[f"mfma_i8_{name}_ms"] = ms
        # the same operands on the tile kernel's pattern (a 128 x 64 piece per wavefront), in both forms of the instruction
        for form in (32, 16):
            def run_tile():
                L.check(lib.omni_diag_mfma_i8_tile_rate(ops_buf.data_ptr(), ops_buf.numel(), form, iters, cus, sink.data_ptr(), st),
                        "omni_diag_mfma_i8_tile_rate")
            ms = ev_ms(run_tile, 5)
            res[f"mfma_i8_tile_pattern_{form}_{name}_pops"] = cus * 8 * iters * 2.0 * 128 * 64 * 64 / (ms * 1e-3) / 1e15
    for tag, (M, K, N) in (("gemm1_shape", (65536, 7168, 4096)), ("gemm2_shape", (65536, 2048, 7168))):
        a = torch.randint(-128, 128, (M, K), generator=g, device=dev, dtype=torch.int8)
        b = torch.randint(-128, 128, (N, K), generator=g, device=dev, dtype=torch.int8).t()   # column-major B
        ms = ev_ms(lambda: torch._int_mm(a, b), 5)
        res[f"vendor_int_mm_{tag}_pops"] = 2.0 * M * K * N / (ms * 1e-3) / 1e15
        res[f"vendor_int_mm_{tag}_us"] = ms * 1e3
        del a, b
    # the library's own tile kernels at the prefill shape, once on the real operands and once on zeros: the
    # same instruction stream at the clock the chip grants each kind of data
    from omni_infer_amd import hip_ops as ops
    cfg = SHAPES["prefill"]
    T, H, I, K, n_local = cfg["T"], cfg["H"], cfg["I"], cfg["K"], cfg["n_local"]
    ws = WeightSet(cfg, 100, dev)
    ws.drop_ckpt()
    x, logits, bias = make_inputs(cfg, dev)
    w, ids, _ = ops.npu_moe_gating_top_k(logits, K, bias, cfg["topk_group"], cfg["n_group"], 1, 0, 1, cfg["scale"], 1e-20)
    p = ops.moe_permute(ids, 0, n_local, L.OMNI_IDX_TOKEN_MAJOR)
    M_cap = T * K + T
    xq, xs = ops.npu_dynamic_quant(x)
    g1_ws = torch.zeros(lib.omni_moe_gemm1_workspace_bytes(T, K, n_local, T, M_cap, H, I), dtype=torch.uint8, device=dev)
    hq = torch.empty(M_cap, I, dtype=torch.int8, device=dev)
    hs = torch.empty(M_cap, dtype=torch.float32, device=dev)
    rows = torch.empty(M_cap, H, dtype=torch.float32, device=dev)

    def g1(flags=L.OMNI_GEMM1_NO_REQUANT):
        ops.grouped_gemm1_swiglu_quant(xq, xs, p.sorted_src, L.OMNI_IDX_TOKEN_MAJOR, K, ws.w13, ws.s13, p.offsets, H, I,
                                       M_cap, extra=(ws.sh13, ws.sh_s13), extra_rows=T, flags=flags, workspace=g1_ws,
                                       out=(hq, hs))

    def g2():
        ops.grouped_gemm2_dequant(hq, hs, ws.w2, ws.s2, p.offsets, H, I, out_dtype=torch.float32,
                                  extra=(ws.sh2, ws.sh_s2), extra_rows=T, out=rows, workspace=g1_ws)

    g1(0)   # real int8 rows for GEMM2
    res["tile_kernels"] = {"gemm1": ops.gemm_kernel_name(1, T, K, n_local, T, M_cap, H, I),
                           "gemm2": ops.gemm_kernel_name(2, T, K, n_local, T, M_cap, H, I), "rows": M_cap}
    res["tile_gemm1_real_operands_us"] = ev_ms(g1, 10) * 1e3
    res["tile_gemm2_real_operands_us"] = ev_ms(g2, 10) * 1e3
    xq.zero_()
    hq.zero_()
    res["tile_gemm1_zero_activations_us"] = ev_ms(g1, 10) * 1e3
    res["tile_gemm2_zero_activations_us"] = ev_ms(g2, 10) * 1e3
    for t in (ws.w13, ws.sh13, ws.w2, ws.sh2):
        t.zero_()
    res["tile_gemm1_zero_operands_us"] = ev_ms(g1, 10) * 1e3
    res["tile_gemm2_zero_operands_us"] = ev_ms(g2, 10) * 1e3
    ops1, ops2 = 2.0 * M_cap * H * 2 * I, 2.0 * M_cap * I * H
    for k in ("real_operands", "zero_operands"):
        res[f"tile_gemm1_{k}_pops"] = ops1 / (res[f"tile_gemm1_{k}_us"] * 1e-6) / 1e15
        res[f"tile_gemm2_{k}_pops"] = ops2 / (res[f"tile_gemm2_{k}_us"] * 1e-6) / 1e15
    del ws, xq, hq, rows, g1_ws
    src = torch.ones(1 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    ms = ev_ms(lambda: dst.copy_(src), 10)
    res["copy_1GiB_read_plus_write_TBps"] = 2 * (1 << 30) / (ms * 1e-3) / 1e12
    # a kernel that only reads (the library's diagnostic): the ceiling of the weight-streaming GEMMs of the decode step
    del dst
    best = (0.0, 0)
    for per_cu in (4, 8, 16, 32, 64):
        def rd():
            L.check(lib.omni_diag_hbm_read_rate(src.data_ptr(), src.numel(), cus * per_cu, sink.data_ptr(), st),
                    "omni_diag_hbm_read_rate")
        tbps = (1 << 30) / (ev_ms(rd, 10) * 1e-3) / 1e12
        res[f"read_1GiB_{per_cu}_blocks_per_cu_TBps"] = tbps
        best = max(best, (tbps, per_cu))
    res["read_1GiB_best_TBps"] = best[0]
    res["value"] = res["mfma_i8_gaussian_sigma30_pops"]
    print(json.dumps(res))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=4000, help="timed decode steps (prefill runs steps/100, at least 10)")
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", choices=["all", "decode", "prefill", "norm", "calib"], default="all",
                    help="all (default): decode headline + prefill object + block_us; decode / prefill: that half only; "
                         "norm: the RMSNorm+quant producer; calib: what the hardware delivers (matrix instruction "
                         "alone, vendor int8 GEMM, copy)")
    ap.add_argument("--rows", choices=["f32", "bf16"], default="f32",
                    help="row dtype between GEMM2 and the combine (the product default is f32)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-block", action="store_true", help="skip the DeepseekMoE.forward timing")
    ap.add_argument("--weight-sets", type=int, default=2, help="weight copies rotated between steps (cache defeat)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run three 1 GiB device copies first (a kernel of known traffic to scale HBM counters by)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU's expert share on one GPU; --gpus must be 1 "
              "(no collectives are part of it)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)

    if args.workload == "calib":
        return bench_calib(args)
    if args.workload == "norm":
        if args.steps == 4000:
            args.steps, args.warmup = 200, 20
        return bench_norm(args)

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    rows_dtype = torch.float32 if args.rows == "f32" else torch.bfloat16
    cfg = SHAPES["decode"]
    sets = [WeightSet(cfg, 100 + i, dev) for i in range(max(1, args.weight_sets))]
    for s in sets[1:]:
        s.drop_ckpt()

    if args.copy_probe:
        src = torch.ones(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    pre_steps = max(10, args.steps // 100)
    dec = pre = None
    if args.workload in ("all", "decode"):
        dec, _ = measure_layer("decode", sets, args.steps, args.warmup, rows_dtype, args.no_cpu, dev)
    if args.workload in ("all", "prefill"):
        pre, _ = measure_layer("prefill", sets, pre_steps, 3, rows_dtype, args.no_cpu, dev, kernel_steps=pre_steps)
        if args.workload == "all":
            other = torch.bfloat16 if rows_dtype == torch.float32 else torch.float32
            alt, _ = measure_layer("prefill", sets, pre_steps, 3, other, True, dev, kernel_steps=pre_steps)
            pre["other_rows_dtype"] = {k: alt[k] for k in ("rows_dtype", "layer_us", "int8_frac")}
            pre["other_rows_dtype"]["gemm2_kernel_us"] = alt["roofline_gemm2"]["kernel_us"]
            pre["global_filter"] = measure_global_filter(sets, max(20, pre_steps), 3, rows_dtype, dev)

    head = dec if dec is not None else pre
    result = {
        "metric": "moe_layer_latency", "value": head["layer_us"], "unit": "us", "n_gpus": 1, "steps": head["steps"],
        "warmup": head["warmup"], "preheat_steps": head["preheat_steps"], "ms_per_step": head["ms_per_step"],
        "graph_us": head["graph_us"], "higher_is_better": False, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": head["workload"], "tokens": head["tokens"], "rows_routed": head["rows_routed"],
                   "active_groups": head["active_groups"], "weight_sets": len(sets), "rows_dtype": head["rows_dtype"]},
        "layer": {k: head[k] for k in ("algorithmic_bytes", "algorithmic_ops", "hbm_frac", "int8_frac",
                                       "host_wall_ms_per_step", "single_step_us")},
        "roofline": head["roofline_gemm1"],
        "roofline_gemm2": head["roofline_gemm2"],
    }
    if "cpu_baseline" in head:
        result["cpu_baseline"] = head["cpu_baseline"]
    if dec is not None and pre is not None:
        result["prefill"] = {k: pre[k] for k in ("workload", "tokens", "rows_routed", "rows_dtype", "layer_us", "steps",
                                                 "preheat_steps",
                                                 "algorithmic_ops", "int8_frac", "single_step_us", "roofline_gemm1",
                                                 "roofline_gemm2", "other_rows_dtype", "global_filter")}
        if "cpu_baseline" in pre:
            result["prefill"]["gpu_vs_oracle_rel_err"] = pre["cpu_baseline"]["gpu_vs_oracle_rel_err"]
            result["prefill"]["gpu_vs_oracle_bit_exact"] = pre["cpu_baseline"]["gpu_vs_oracle_bit_exact"]
            result["prefill"]["cpu_baseline"] = pre["cpu_baseline"]
    if not args.no_block and args.workload == "all":
        result["block_us"] = {"decode": measure_block("decode", sets[0], max(50, args.steps // 10), 10, dev),
                              "prefill": measure_block("prefill", sets[0], pre_steps, 2, dev)}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
