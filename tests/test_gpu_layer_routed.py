"""Router and layer in one library call against the router's call followed by the layer's: the same bits
(output, routing weights, ids), on calls that route, quantise and sort in a single launch and on calls that do
not fit that kernel."""
import pytest
import torch

from tests.helpers import Layer, gen, tokens

pytestmark = pytest.mark.gpu


def _route_args(E, mode):
    from omni_infer_amd import _lib as L
    if mode == "noaux_tc":      # sigmoid + bias, groups by the sum of their two best (layer.py:341-351)
        return dict(top_k=8, n_group=8, topk_group=4, score_fn="sigmoid", group_mode=L.OMNI_GROUP_TOP2SUM,
                    masked_fill_zero=False, weight_from_c=False, renorm=True, scale=2.5, eps=1e-20)
    if mode == "softmax":       # fused_topk (fused_moe.py:24-34)
        return dict(top_k=2, n_group=1, topk_group=1, score_fn="softmax", group_mode=L.OMNI_GROUP_MAX,
                    masked_fill_zero=False, weight_from_c=False, renorm=True, scale=1.0, eps=0.0)
    raise AssertionError(mode)


def _both(x, logits, bias, ra, lo, n, d, shared, H, I, rows_dtype=torch.float32, x_scale=None):
    from omni_infer_amd import hip_ops as ops
    w, ids = ops.moe_route(logits, bias, **ra)
    want = ops.moe_w8a8_layer(x, x_scale, w, ids, lo, lo + n, d["w13"], d["s13"], d["w2"], d["s2"], shared, H=H, I=I,
                              rows_dtype=rows_dtype)
    got, gw, gids = ops.moe_w8a8_layer_routed(x, x_scale, logits, bias, lo=lo, hi=lo + n, w13_packed=d["w13"],
                                              w13_scale=d["s13"], w2_packed=d["w2"], w2_scale=d["s2"], shared=shared,
                                              H=H, I=I, rows_dtype=rows_dtype, **ra)
    torch.cuda.synchronize()
    return (want, w, ids), (got, gw, gids)


def _same(a, b, what):
    for u, v, name in zip(a, b, ("output", "routing weights", "ids")):
        assert torch.equal(u, v), f"{what}: {name} differ"


@pytest.mark.parametrize("T", [1, 3, 64, 130, 512])
def test_single_launch_front_matches_two_calls(T):
    """E=256 in 8 groups, top 8 of the 4 best groups, 32 local experts from id 64: the decode-sized calls whose
    first launch routes, quantises and sorts.  Token counts that are not multiples of four leave routing
    wavefronts without a token; every call reuses an arrival counter that an earlier call left behind."""
    E, n, H, I, lo = 256, 32, 1024, 256, 64
    lay = Layer(n, H, I, seed=401, shared=True)
    d = lay.to_device()
    shared = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"])
    g = gen(402 + T)
    ra = _route_args(E, "noaux_tc")
    for rep in range(3):
        x = tokens(T, H, 403 + rep).cuda()
        logits = torch.randn(T, E, generator=g).cuda()
        bias = (torch.randn(E, generator=g) * 0.1).cuda()
        a, b = _both(x, logits, bias, ra, lo, n, d, shared, H, I)
        _same(a, b, f"T={T} call {rep}")
        assert bool(((a[2] >= lo) & (a[2] < lo + n)).any()) or T < 3


def test_many_calls_in_a_row_reuse_the_counters():
    """More calls than the library holds arrival counters: each counter is used again and must have been left
    at zero by the call that used it before."""
    E, n, H, I = 8, 8, 1024, 512
    lay = Layer(n, H, I, seed=411, shared=False)
    d = lay.to_device()
    g = gen(412)
    ra = _route_args(E, "softmax")
    T = 37
    x = tokens(T, H, 413).cuda()
    logits = torch.randn(T, E, generator=g).cuda()
    a, b = _both(x, logits, None, ra, 0, n, d, None, H, I)
    _same(a, b, "first call")
    from omni_infer_amd import hip_ops as ops
    out = torch.empty_like(a[0])
    for i in range(600):
        ops.moe_w8a8_layer_routed(x, None, logits, None, lo=0, hi=n, w13_packed=d["w13"], w13_scale=d["s13"],
                                  w2_packed=d["w2"], w2_scale=d["s2"], shared=None, H=H, I=I, out=out, **ra)
        if i % 97 == 0:
            torch.cuda.synchronize()
            assert torch.equal(out, a[0]), f"call {i}"
            out.zero_()
    torch.cuda.synchronize()
    assert torch.equal(out, a[0])


@pytest.mark.parametrize("case", ["many_tokens", "int8_tokens", "bf16_rows"])
def test_calls_outside_the_single_launch_front(case):
    """More than 4096 assignments, or tokens that arrive quantised: the router runs as a launch of its own and the
    results are still those of the two calls."""
    E, n, H, I, lo = 64, 16, 512, 256, 8
    lay = Layer(n, H, I, seed=421, shared=True)
    d = lay.to_device()
    shared = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"])
    g = gen(422)
    ra = _route_args(E, "noaux_tc")
    T = 700 if case == "many_tokens" else 48
    x = tokens(T, H, 423).cuda()
    logits = torch.randn(T, E, generator=g).cuda()
    bias = (torch.randn(E, generator=g) * 0.1).cuda()
    xs = None
    if case == "int8_tokens":
        from omni_infer_amd import hip_ops as ops
        x, xs = ops.npu_dynamic_quant(x)
    rows_dtype = torch.bfloat16 if case == "bf16_rows" else torch.float32
    a, b = _both(x, logits, bias, ra, lo, n, d, shared, H, I, rows_dtype=rows_dtype, x_scale=xs)
    _same(a, b, case)


def test_routed_entry_rejects_bad_routing_arguments():
    from omni_infer_amd import hip_ops as ops
    E, n, H, I = 64, 16, 512, 256
    lay = Layer(n, H, I, seed=431, shared=False)
    d = lay.to_device()
    x = tokens(8, H, 432).cuda()
    logits = torch.zeros(8, E, device="cuda")
    ra = _route_args(E, "noaux_tc")
    ra["n_group"] = 7   # does not divide 64
    with pytest.raises(RuntimeError, match="n_group"):
        ops.moe_w8a8_layer_routed(x, None, logits, None, lo=0, hi=n, w13_packed=d["w13"], w13_scale=d["s13"],
                                  w2_packed=d["w2"], w2_scale=d["s2"], shared=None, H=H, I=I, **ra)
    with pytest.raises(ValueError, match="one row of logits per token"):
        ops.moe_w8a8_layer_routed(x, None, logits[:4], None, lo=0, hi=n, w13_packed=d["w13"], w13_scale=d["s13"],
                                  w2_packed=d["w2"], w2_scale=d["s2"], shared=None, H=H, I=I,
                                  **_route_args(E, "noaux_tc"))


def test_routed_call_is_graph_capturable():
    """The routed entry captured in a HIP graph and replayed with eager work in between: the arrival counter a
    capture took is left at zero by every replay."""
    E, n, H, I, K, T = 32, 4, 1024, 512, 8, 64
    from omni_infer_amd import _lib as L
    from omni_infer_amd import hip_ops as ops
    lay = Layer(n, H, I, seed=441, shared=True)
    d = lay.to_device()
    shared = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"])
    g = gen(442)
    x = tokens(T, H, 443).cuda()
    logits = torch.randn(T, E, generator=g).cuda()
    bias = (torch.randn(E, generator=g) * 0.01).cuda()
    ra = _route_args(E, "noaux_tc")
    need = L.lib().omni_moe_w8a8_layer_workspace_bytes(T, K, n, H, I, 1, L.OMNI_DT_F32)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    out = torch.empty(T, H, dtype=torch.bfloat16, device="cuda")
    tw = torch.empty(T, K, dtype=torch.float32, device="cuda")
    ti = torch.empty(T, K, dtype=torch.int32, device="cuda")

    def step():
        return ops.moe_w8a8_layer_routed(x, None, logits, bias, lo=0, hi=n, w13_packed=d["w13"], w13_scale=d["s13"],
                                         w2_packed=d["w2"], w2_scale=d["s2"], shared=shared, H=H, I=I, workspace=ws,
                                         out=out, topk_w=tw, topk_ids=ti, **ra)[0]

    eager = step().clone()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        step()
    for rep in range(3):
        out.zero_()
        ti.zero_()
        junk = torch.randn(256, 256, device="cuda") @ torch.randn(256, 256, device="cuda")
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {rep} differs from the eager run"
        del junk
    x.copy_(tokens(T, H, 444).cuda())
    logits.copy_(torch.randn(T, E, generator=g).cuda())
    graph.replay()
    torch.cuda.synchronize()
    replayed = out.clone()
    assert torch.equal(step(), replayed), "replay on new inputs differs from the eager run"


@pytest.mark.parametrize("T", [300, 777])
def test_layer_entry_matches_the_separate_operators_at_tile_sizes(T):
    """The layer entry against quantise, sort, GEMM1, GEMM2 and weighted sum called one by one, where both grouped
    GEMMs run the tile kernel: inside the entry the shared expert's rows go from GEMM2 to the weighted sum as bf16
    (packed into the front half of their fp32 place), outside they stay fp32 and are rounded by the weighted sum;
    the bits must be the same.  The token counts leave a last row block of 44 and of 9 shared rows."""
    from omni_infer_amd import _lib as L
    from omni_infer_amd import hip_ops as ops
    H, I, n, E, K, lo = 1024, 512, 8, 16, 4, 3
    lay = Layer(n, H, I, seed=451, shared=True)
    d = lay.to_device()
    shared = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"])
    g = gen(452 + T)
    x = tokens(T, H, 453).cuda()
    ids = torch.rand(T, E, generator=g).argsort(dim=1)[:, :K].to(torch.int32).cuda()
    w = torch.rand(T, K, generator=g).cuda()
    assert "gemm_pipe" in ops.gemm_kernel_name(2, T, K, n, T, T * K + T, H, I)
    got = ops.moe_w8a8_layer(x, None, w, ids, lo, lo + n, d["w13"], d["s13"], d["w2"], d["s2"], shared, H=H, I=I)

    xq, xs = ops.npu_dynamic_quant(x)
    p = ops.moe_permute(ids, lo, lo + n, L.OMNI_IDX_TOKEN_MAJOR)
    M_cap = T * K + T
    hq, hs, _ = ops.grouped_gemm1_swiglu_quant(xq, xs, p.sorted_src, L.OMNI_IDX_TOKEN_MAJOR, K, d["w13"], d["s13"],
                                               p.offsets, H, I, M_cap, extra=(d["sh13"], d["sh_s13"]), extra_rows=T)
    rows, _ = ops.grouped_gemm2_dequant(hq, hs, d["w2"], d["s2"], p.offsets, H, I, out_dtype=torch.float32,
                                        extra=(d["sh2"], d["sh_s2"]), extra_rows=T)
    want = ops.moe_combine(rows, w, p.src_to_dst, L.OMNI_IDX_TOKEN_MAJOR, L.OMNI_ORDER_SLOT, post_add=rows,
                           post_add_row0=p.offsets[n:])
    torch.cuda.synchronize()
    assert torch.equal(got, want)


def test_routed_calls_on_two_streams_do_not_share_a_counter():
    """Two streams, each with its own workspace and outputs, issue routed calls without waiting for each other: calls
    in flight at the same time hold different arrival counters, so both streams get the bits of a call made alone."""
    from omni_infer_amd import _lib as L
    from omni_infer_amd import hip_ops as ops
    E, n, H, I, K = 32, 4, 1024, 512, 8
    lay = Layer(n, H, I, seed=461, shared=True)
    d = lay.to_device()
    shared = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"])
    ra = _route_args(E, "noaux_tc")
    g = gen(462)
    jobs = []
    for T in (64, 47):
        x = tokens(T, H, 463 + T).cuda()
        logits = torch.randn(T, E, generator=g).cuda()
        bias = (torch.randn(E, generator=g) * 0.01).cuda()
        need = L.lib().omni_moe_w8a8_layer_workspace_bytes(T, K, n, H, I, 1, L.OMNI_DT_F32)
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        out = torch.empty(T, H, dtype=torch.bfloat16, device="cuda")
        tw = torch.empty(T, K, dtype=torch.float32, device="cuda")
        ti = torch.empty(T, K, dtype=torch.int32, device="cuda")
        kw = dict(lo=0, hi=n, w13_packed=d["w13"], w13_scale=d["s13"], w2_packed=d["w2"], w2_scale=d["s2"], shared=shared,
                  H=H, I=I, workspace=ws, out=out, topk_w=tw, topk_ids=ti, **ra)
        alone = ops.moe_w8a8_layer_routed(x, None, logits, bias, **kw)[0].clone()
        jobs.append((x, logits, bias, kw, out, alone, torch.cuda.Stream()))
    torch.cuda.synchronize()
    for rep in range(40):
        for x, logits, bias, kw, out, alone, stream in jobs:
            with torch.cuda.stream(stream):
                ops.moe_w8a8_layer_routed(x, None, logits, bias, **kw)
    torch.cuda.synchronize()
    for x, logits, bias, kw, out, alone, stream in jobs:
        assert torch.equal(out, alone)


@pytest.mark.parametrize("E,n_group,topk_group,K", [(40, 1, 1, 4), (384, 8, 3, 6), (512, 4, 2, 8)])
def test_single_launch_front_with_other_expert_counts(E, n_group, topk_group, K):
    """Expert counts that give a lane 1, 6 and 8 experts (40 leaves lanes without an expert), with and without
    groups; the local range lies where only part of the assignments fall into it."""
    from omni_infer_amd import _lib as L
    n, H, I, lo, T = 8, 512, 256, 16, 50
    lay = Layer(n, H, I, seed=471, shared=True)
    d = lay.to_device()
    shared = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"])
    g = gen(472 + E)
    ra = dict(top_k=K, n_group=n_group, topk_group=topk_group, score_fn="sigmoid", group_mode=L.OMNI_GROUP_TOP2SUM,
              masked_fill_zero=False, weight_from_c=False, renorm=True, scale=2.5, eps=1e-20)
    x = tokens(T, H, 473).cuda()
    logits = torch.randn(T, E, generator=g).cuda()
    bias = (torch.randn(E, generator=g) * 0.1).cuda()
    a, b = _both(x, logits, bias, ra, lo, n, d, shared, H, I)
    _same(a, b, f"E={E}")


def test_routed_entry_when_nothing_is_local_and_when_there_are_no_tokens():
    """No assignment falls into the local range: the output is the shared expert's alone (and zero without one).
    No tokens: the call returns without launching anything."""
    from omni_infer_amd import hip_ops as ops
    E, n, H, I, lo, T = 64, 8, 512, 256, 56, 24
    lay = Layer(n, H, I, seed=481, shared=True)
    d = lay.to_device()
    shared = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"])
    ra = _route_args(E, "noaux_tc")
    g = gen(482)
    x = tokens(T, H, 483).cuda()
    logits = torch.randn(T, E, generator=g)
    logits[:, lo:lo + n] = -30.0            # the local experts are never chosen
    logits = logits.cuda()
    a, b = _both(x, logits, None, ra, lo, n, d, shared, H, I)
    _same(a, b, "nothing local, shared expert")
    assert not bool(((a[2] >= lo) & (a[2] < lo + n)).any())
    a, b = _both(x, logits, None, ra, lo, n, d, None, H, I)
    _same(a, b, "nothing local, no shared expert")
    assert not bool(b[0].float().abs().any())
    out, w, ids = ops.moe_w8a8_layer_routed(x[:0], None, logits[:0], None, lo=lo, hi=lo + n, w13_packed=d["w13"],
                                            w13_scale=d["s13"], w2_packed=d["w2"], w2_scale=d["s2"], shared=shared,
                                            H=H, I=I, **ra)
    assert tuple(out.shape) == (0, H) and tuple(ids.shape) == (0, 8)


# ----------------------------------------------------------------------------- the whole block in one call
def _block_both(x, gate_w, bias, ra, lo, n, d, shared, H, I, rows_dtype=torch.float32, quantised=False):
    """gate + router (one call) followed by the layer (one call), against the block entry."""
    from omni_infer_amd import hip_ops as ops
    bf16_gate = gate_w.dtype == torch.bfloat16
    w, ids, _ = ops.moe_gate_route(x, gate_w, bias, ra["top_k"], ra["n_group"], ra["topk_group"], ra["score_fn"],
                                   ra["group_mode"], ra["masked_fill_zero"], ra["weight_from_c"], ra["renorm"], ra["scale"],
                                   ra["eps"], round_logits_bf16=bf16_gate)
    xq = xs = None
    if quantised:
        xq, xs = ops.npu_dynamic_quant(x)
    want = ops.moe_w8a8_layer(xq if quantised else x, xs, w, ids, lo, lo + n, d["w13"], d["s13"], d["w2"], d["s2"], shared,
                              H=H, I=I, rows_dtype=rows_dtype)
    got, gw, gids = ops.moe_w8a8_block(x, gate_w, bias, lo=lo, hi=lo + n, w13_packed=d["w13"], w13_scale=d["s13"],
                                       w2_packed=d["w2"], w2_scale=d["s2"], shared=shared, H=H, I=I, x_int8=xq,
                                       pertoken_scale=xs, round_logits_bf16=bf16_gate, rows_dtype=rows_dtype, **ra)
    torch.cuda.synchronize()
    return (want, w, ids), (got, gw, gids)


@pytest.mark.parametrize("T", [1, 5, 64, 128, 200])
@pytest.mark.parametrize("quantised", [False, True])
def test_block_entry_matches_gate_route_then_layer(T, quantised):
    """E=256 in 8 groups, top 8, 32 local experts from id 64, H=1024: up to 128 tokens the launch behind the gate's
    partial sums adds them up, routes, quantises and sorts; 200 tokens (1600 assignments) take the separate
    launches.  With tokens that arrive quantised that launch has no quantising blocks."""
    E, n, H, I, lo = 256, 32, 1024, 256, 64
    lay = Layer(n, H, I, seed=501, shared=True)
    d = lay.to_device()
    shared = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"])
    g = gen(502 + T)
    ra = _route_args(E, "noaux_tc")
    gate_w = (torch.randn(E, H, generator=g) * 0.05).cuda()
    for rep in range(2):
        x = tokens(T, H, 503 + rep).cuda()
        bias = (torch.randn(E, generator=g) * 0.1).cuda()
        a, b = _block_both(x, gate_w, bias, ra, lo, n, d, shared, H, I, quantised=quantised)
        _same(a, b, f"T={T} quantised={quantised} call {rep}")


@pytest.mark.parametrize("case", ["bf16_gate", "softmax_top2", "no_shared_bf16_rows", "wide_H"])
def test_block_entry_variants(case):
    from omni_infer_amd import _lib as L
    E, n, H, I, lo, T = 64, 16, 512, 256, 8, 48
    shared_on, rows_dtype, gdt = True, torch.float32, torch.float32
    ra = dict(top_k=8, n_group=8, topk_group=4, score_fn="sigmoid", group_mode=L.OMNI_GROUP_TOP2SUM,
              masked_fill_zero=False, weight_from_c=False, renorm=True, scale=2.5, eps=1e-20)
    if case == "bf16_gate":
        gdt = torch.bfloat16
    elif case == "softmax_top2":
        E, n, lo = 8, 8, 0
        ra = _route_args(E, "softmax")
    elif case == "no_shared_bf16_rows":
        shared_on, rows_dtype = False, torch.bfloat16
    elif case == "wide_H":
        H = 7168          # 56 slices of the gate projection: 7 groups of partial sums
    lay = Layer(n, H, I, seed=511, shared=shared_on)
    d = lay.to_device()
    shared = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"]) if shared_on else None
    g = gen(512)
    gate_w = (torch.randn(E, H, generator=g) * 0.05).to(gdt).cuda()
    bias = (torch.randn(E, generator=g) * 0.1).cuda() if ra["score_fn"] == "sigmoid" else None
    x = tokens(T, H, 513).cuda()
    a, b = _block_both(x, gate_w, bias, ra, lo, n, d, shared, H, I, rows_dtype=rows_dtype)
    _same(a, b, case)


def test_block_entry_under_graph_capture_and_replay():
    """The block entry recorded into a HIP graph (its arrival counter then comes from the pool that eager calls
    never use) and replayed with eager calls of the routed entry in between: every replay gives the eager bits."""
    from omni_infer_amd import hip_ops as ops
    E, n, H, I, lo, T = 256, 32, 1024, 256, 0, 24
    lay = Layer(n, H, I, seed=521, shared=True)
    d = lay.to_device()
    shared = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"])
    g = gen(522)
    ra = _route_args(E, "noaux_tc")
    gate_w = (torch.randn(E, H, generator=g) * 0.05).cuda()
    bias = (torch.randn(E, generator=g) * 0.1).cuda()
    x = tokens(T, H, 523).cuda()
    K = ra["top_k"]
    need = ops.L.lib().omni_moe_w8a8_block_workspace_bytes(T, K, n, H, I, E, 1, ops.L.OMNI_DT_F32)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    out = torch.empty(T, H, dtype=torch.bfloat16, device="cuda")
    tw = torch.empty(T, K, dtype=torch.float32, device="cuda")
    ti = torch.empty(T, K, dtype=torch.int32, device="cuda")

    def call():
        ops.moe_w8a8_block(x, gate_w, bias, lo=lo, hi=lo + n, w13_packed=d["w13"], w13_scale=d["s13"], w2_packed=d["w2"],
                           w2_scale=d["s2"], shared=shared, H=H, I=I, workspace=ws, out=out, topk_w=tw, topk_ids=ti, **ra)
    call()
    torch.cuda.synchronize()
    want, want_ids = out.clone(), ti.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            call()
            call()
    torch.cuda.current_stream().wait_stream(side)
    logits = torch.randn(T, E, generator=g).cuda()
    for rep in range(5):
        out.zero_()
        ti.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want) and torch.equal(ti, want_ids), f"replay {rep}"
        # eager work between the replays, through the counters of the eager pool
        ops.moe_w8a8_layer_routed(x, None, logits, bias, lo=lo, hi=lo + n, w13_packed=d["w13"], w13_scale=d["s13"],
                                  w2_packed=d["w2"], w2_scale=d["s2"], shared=shared, H=H, I=I, **ra)
        torch.cuda.synchronize()
