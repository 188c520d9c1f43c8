"""Whole-pipeline parity on the GPU: the reference's quant-method / layer / block surface over the
HIP library against the CPU oracle, on the five benchmark configurations (reduced expert counts
where the full one would not fit the test budget, real widths), plus size-independent
properties at the full benchmark sizes."""
import types

import pytest
import torch

from oracle import moe_oracle as O
from tests.helpers import Layer, cosine, gen, rel_err, tokens

pytestmark = pytest.mark.gpu

REL_TOL, COS_TOL = 1e-2, 0.9995   # the stated bar for bf16 outputs


@pytest.fixture(scope="module")
def env():
    assert torch.cuda.is_available()
    from omni_infer_amd import _lib as L
    from omni_infer_amd import hip_ops as ops
    from omni_infer_amd import config, distributed
    return types.SimpleNamespace(L=L, ops=ops, config=config, dist=distributed)


def _check_out(got, want, exact=True):
    got, want = got.float().cpu(), want.float().cpu()
    r, c = rel_err(got, want), cosine(got, want)
    assert r <= REL_TOL and c >= COS_TOL, f"rel_err {r:.3e} cosine {c:.6f}"
    if exact:
        assert torch.equal(got, want), f"within tolerance (rel {r:.2e}) but not bit exact"


def _make_fused_moe(env, lay, E_total, K, ep_size, rank, grouped=None, scoring="softmax", bias=None, renorm=True):
    from omni_infer_amd.layers.layer import FusedMoE
    from omni_infer_amd.quantization.compressed_tensors import AscendCompressedTensorsConfig
    env.dist.set_virtual_ep(ep_size, rank)
    kw = {}
    if grouped:
        kw = dict(use_grouped_topk=True, num_expert_group=grouped[0], topk_group=grouped[1])
    m = FusedMoE(num_experts=E_total, top_k=K, hidden_size=lay.H, intermediate_size=lay.I,
                 params_dtype=torch.bfloat16, renormalize=renorm, quant_config=AscendCompressedTensorsConfig(),
                 scoring_func=scoring, e_score_correction_bias=bias, device="cuda", **kw)
    lo = rank * lay.n_local if env.config.model_extra_config.operator_opt_config.enable_moe_expert_parallel else 0
    # feed the checkpoint tensors through the layer's own weight_loader, expert by expert
    for e in range(lay.n_local):
        ge = lo + e
        m.weight_loader(m.w13_weight, lay.w13_ckpt[e, :lay.I], "experts.w13_weight", "w1", ge)
        m.weight_loader(m.w13_weight, lay.w13_ckpt[e, lay.I:], "experts.w13_weight", "w3", ge)
        m.weight_loader(m.w2_weight, lay.w2_ckpt[e], "experts.w2_weight", "w2", ge)
        m.weight_loader(m.w13_weight_scale, lay.s13[e, :lay.I].unsqueeze(-1), "experts.w13_weight_scale", "w1", ge)
        m.weight_loader(m.w13_weight_scale, lay.s13[e, lay.I:].unsqueeze(-1), "experts.w13_weight_scale", "w3", ge)
        m.weight_loader(m.w2_weight_scale, lay.s2[e].unsqueeze(-1), "experts.w2_weight_scale", "w2", ge)
    return m


def _bf16_scales(lay):
    # create_weights keeps scales in bf16 parameters for a bf16 model (compressed_tensors_moe.py:64-68):
    # what the layer computes with is the bf16-rounded scale, so the oracle gets the same
    lay.s13 = lay.s13.to(torch.bfloat16).float()
    lay.s2 = lay.s2.to(torch.bfloat16).float()
    return lay


# ------------------------------------------------------------------ config 1: toy layer, non-EP apply()
def test_config1_toy_apply_non_ep(env):
    """8 experts, H=1024, I=512, top-2 softmax renormalised, 64 tokens, no shared expert:
    quant_method.apply() in its non-EP branch = fused_experts_w8a8 (bf16 between the stages)."""
    env.config.update_model_extra_config(enable_moe_expert_parallel=False)
    try:
        lay = _bf16_scales(Layer(8, 1024, 512, seed=0))
        m = _make_fused_moe(env, lay, 8, 2, 1, 0)
        m.quant_method.process_weights_after_loading(m)
        g = gen(0)
        x = tokens(64, 1024, 0)
        gate = (torch.randn(8, 1024, generator=g) * 0.02).to(torch.bfloat16)
        logits = x.float() @ gate.float().t()
        w_ref, id_ref, row_ref = O.route_softmax_topk(logits, 2, True)
        out_ref, st = O.fused_experts_w8a8(x, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w_ref, id_ref, row_ref,
                                           return_stages=True)
        w, ids, row = m.select_experts(x.cuda(), logits.cuda(), 2, False, True)
        assert torch.equal(ids.cpu(), id_ref) and torch.equal(w.cpu(), w_ref)
        out = m(x.cuda(), w, ids, None, None)
        _check_out(out, out_ref)
    finally:
        env.config.update_model_extra_config(enable_moe_expert_parallel=True)


def test_config1_toy_one_rank_dispatch_combine(env):
    """Same toy layer through the dispatch/combine branch in its one-rank form."""
    env.config.update_model_extra_config(enable_moe_expert_parallel=True, moe_dispatch_combine=True,
                                         prefill_dispatch_combine=True)
    lay = Layer(8, 1024, 512, seed=0)
    m = _make_fused_moe(env, _bf16_scales(lay), 8, 2, 1, 0)
    m.quant_method.process_weights_after_loading(m)
    x = tokens(64, 1024, 1)
    logits = torch.randn(64, 8, generator=gen(1))
    w_ref, id_ref, _ = O.route_softmax_topk(logits, 2, True)
    xq, xs = O.dynamic_quant(x)
    rows, idx, counts, sc = O.moe_init_routing_v2(xq, id_ref, xs, (0, 8))
    rows_out = O.moe_expert_quant_forward(rows, lay.w1_t, lay.w2_t, lay.s13, lay.s2, counts, sc, w2_scale_bf16=True)
    s2d = torch.empty(128, dtype=torch.int32)
    s2d[idx.long()] = torch.arange(128, dtype=torch.int32)
    out_ref = O.moe_finalize_routing(rows_out, None, w_ref, s2d, drop_pad_mode=2)
    out = m(x.cuda(), w_ref.cuda(), id_ref.cuda(), None, None)
    _check_out(out, out_ref)


# ------------------------------------------------------------------ config 2: DeepSeek-V3 shape, decode
def _dsv3_block(env, n_local, ep_size, rank, H=7168, I=2048, seed=3, shared=True):
    """A DeepseekMoE block holding `n_local` of n_local*ep_size experts at DeepSeek-V3 widths."""
    from omni_infer_amd.layers.deepseek_moe import DeepseekMoE
    from omni_infer_amd.quantization.compressed_tensors import AscendCompressedTensorsConfig
    env.config.update_model_extra_config(enable_moe_expert_parallel=True, moe_dispatch_combine=False,
                                         prefill_dispatch_combine=False)
    env.dist.set_virtual_ep(ep_size, rank)
    E = n_local * ep_size
    cfg = types.SimpleNamespace(hidden_size=H, n_routed_experts=E, num_experts_per_tok=8, moe_intermediate_size=I,
                                n_shared_experts=1 if shared else None, n_group=8, topk_group=4, norm_topk_prob=True,
                                scoring_func="sigmoid", topk_method="noaux_tc", routed_scaling_factor=2.5,
                                hidden_act="silu", first_k_dense_replace=3)
    blk = DeepseekMoE(cfg, AscendCompressedTensorsConfig(ignore=["gate"]), prefix="model.layers.3.mlp", device="cuda")
    lay = _bf16_scales(Layer(n_local, H, I, seed=seed, shared=shared))
    g = gen(seed + 50)
    gate_w = torch.randn(E, H, generator=g) * 0.02
    bias = torch.randn(E, generator=g) * 0.01
    blk.gate.weight.data.copy_(gate_w)
    blk.gate.e_score_correction_bias.data.copy_(bias)
    lo = rank * n_local
    ex = blk.experts
    for e in range(n_local):
        ex.weight_loader(ex.w13_weight, lay.w13_ckpt[e, :I], "w13_weight", "w1", lo + e)
        ex.weight_loader(ex.w13_weight, lay.w13_ckpt[e, I:], "w13_weight", "w3", lo + e)
        ex.weight_loader(ex.w2_weight, lay.w2_ckpt[e], "w2_weight", "w2", lo + e)
        ex.weight_loader(ex.w13_weight_scale, lay.s13[e, :I].unsqueeze(-1), "w13_weight_scale", "w1", lo + e)
        ex.weight_loader(ex.w13_weight_scale, lay.s13[e, I:].unsqueeze(-1), "w13_weight_scale", "w3", lo + e)
        ex.weight_loader(ex.w2_weight_scale, lay.s2[e].unsqueeze(-1), "w2_weight_scale", "w2", lo + e)
    if shared:
        lay.sh_s13 = lay.sh_s13.to(torch.bfloat16).float()
        lay.sh_s2 = lay.sh_s2.to(torch.bfloat16).float()
        lay.shared = (lay.shared[0], lay.sh_s13, lay.shared[2], lay.sh_s2)
        se = blk.shared_experts
        se.gate_up_proj.weight.data.copy_(lay.sh13_ckpt)
        se.gate_up_proj.weight_scale.data.copy_(lay.sh_s13.unsqueeze(-1))
        se.down_proj.weight.data.copy_(lay.sh2_ckpt)
        se.down_proj.weight_scale.data.copy_(lay.sh_s2.unsqueeze(-1))
    blk.process_weights_after_loading()
    return blk, lay, gate_w, bias, lo


def _block_reference(lay, x, logits, bias, lo, n_local):
    return O.deepseek_moe_forward(x, logits, bias, (lay.w1_t, lay.s13, lay.w2_t, lay.s2), lay.shared, 8, 8, 4, 2.5,
                                  (lo, lo + n_local), return_stages=True)


@pytest.mark.parametrize("T,rank", [(64, 0), (64, 5), (1, 2)])
def test_config2_dsv3_decode_block(env, T, rank):
    """DeepSeek-V3 widths, 4 local experts of 32 (8 groups of 4, top-4 groups, top-8), shared expert,
    64 tokens; the block's forward (fused and operator-by-operator) against the oracle.  The gate
    logits are computed once on the GPU and shared with the oracle so that the fp32 summation
    order of the gate GEMM does not enter routing parity."""
    blk, lay, gate_w, bias, lo = _dsv3_block(env, 4, 8, rank)
    x = tokens(T, 7168, 7 + T)
    xd = x.cuda()
    logits = blk.gate(xd.float())[0]
    out_ref, st = _block_reference(lay, x, logits.cpu(), bias, lo, 4)
    w, ids = blk._route(xd)
    assert torch.equal(ids.cpu(), st["topk_ids"]), "routing ids"
    assert torch.equal(w.cpu(), st["topk_w"]), "routing weights"
    out, res = blk(xd, None, None, 3)
    _check_out(out, out_ref)
    blk.fused = False
    out2, _ = blk(xd, None, None, 3)
    _check_out(out2, out_ref)


def test_config2_apply_allgather_ep_int8_input(env):
    """quant_method.apply() in the all-gather expert-parallel branch: int8 tokens + per-token scales in,
    global expert ids, only the local range computed (fused_experts_w8a8_allgather_ep)."""
    env.config.update_model_extra_config(enable_moe_expert_parallel=True, moe_dispatch_combine=False,
                                         prefill_dispatch_combine=False)
    lay = _bf16_scales(Layer(4, 7168, 2048, seed=11))
    m = _make_fused_moe(env, lay, 32, 8, 8, 3, grouped=(8, 4), scoring="sigmoid", bias=torch.zeros(32).cuda())
    m.quant_method.process_weights_after_loading(m)
    g = gen(12)
    x = tokens(48, 7168, 12)
    xq, xs = O.dynamic_quant(x)
    ids = torch.rand(48, 32, generator=g).argsort(dim=1)[:, :8].to(torch.int32)
    w = torch.rand(48, 8, generator=g)
    out_ref = O.fused_experts_w8a8_allgather_ep(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, (12, 16))
    out = m(xq.cuda(), w.cuda(), ids.cuda(), xs.cuda(), None)
    _check_out(out, out_ref)
    # the reference has no result when the share is the whole model (fused_moe.py:504)
    env.dist.set_virtual_ep(1, 0)
    assert m(xq.cuda(), w.cuda(), ids.cuda(), xs.cuda(), None) is None
    env.dist.set_virtual_ep(8, 3)


# ------------------------------------------------------------------ config 3: prefill-sized, outliers
def test_config3_prefill_outliers_reduced(env):
    """DeepSeek-V3 widths, 2 local experts of 16, 1024 tokens with 0.1 % outlier channels x50: the
    tile kernel path end to end against the oracle."""
    lay = Layer(2, 7168, 2048, seed=21, shared=True)
    d = lay.to_device()
    x = tokens(1024, 7168, 21, outlier_frac=0.001)
    g = gen(22)
    ids = (torch.rand(1024, 2, generator=g).argsort(dim=1)[:, :2] + 6).to(torch.int32)   # both local experts
    ids = torch.cat([ids, torch.randint(8, 16, (1024, 2), generator=g).to(torch.int32)], dim=1)  # + 2 remote
    w = torch.rand(1024, 4, generator=g)
    xq, xs = O.dynamic_quant(x)
    out_ref = O.fused_experts_w8a8_allgather_ep(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, (6, 8))
    out_ref = out_ref + O.shared_expert_mlp(x, *lay.shared)
    out = env.ops.moe_w8a8_layer(x.cuda(), None, w.cuda(), ids.cuda(), 6, 8, d["w13"], d["s13"], d["w2"], d["s2"],
                                 (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"]), H=7168, I=2048)
    _check_out(out, out_ref)


# ------------------------------------------------------------------ across the kernel choice
@pytest.mark.parametrize("T,shared", [(80, True), (90, True), (100, True), (96, False), (104, False), (120, False)])
def test_layer_across_the_kernel_crossover(env, T, shared):
    """8 local experts, top-4 among them: T / 2 expected rows per expert.  80 tokens with the shared expert: both
    GEMMs stream (64-row blocks whose bodies take two, three or four tiles by their row count); 90: GEMM1
    streams, GEMM2 (whose groups count the shared rows) runs tiles; 100: both run tiles.  Without the shared expert,
    96: both stream; 104: GEMM1 runs tiles, GEMM2 streams; 120: both tiles.  Every one against the oracle, bit exact."""
    n_local, K, H, I = 8, 4, 1024, 512
    names = {(80, True): ("gemm_stream", "gemm_stream"), (90, True): ("gemm_stream", "gemm_pipe"),
             (100, True): ("gemm_pipe", "gemm_pipe"), (96, False): ("gemm_stream", "gemm_stream"),
             (104, False): ("gemm_pipe", "gemm_stream"), (120, False): ("gemm_pipe", "gemm_pipe")}[(T, shared)]
    M_cap = T * K + (T if shared else 0)
    got_names = (env.ops.gemm_kernel_name(1, T, K, n_local, T if shared else 0, M_cap, H, I),
                 env.ops.gemm_kernel_name(2, T, K, n_local, T if shared else 0, M_cap, H, I))
    assert got_names[0].startswith(names[0]) and got_names[1].startswith(names[1]), got_names
    lay = Layer(n_local, H, I, seed=51, shared=shared)
    d = lay.to_device()
    g = gen(52 + T)
    x = tokens(T, H, 53 + T)
    ids = torch.rand(T, n_local, generator=g).argsort(dim=1)[:, :K].to(torch.int32)
    w = torch.rand(T, K, generator=g)
    xq, xs = O.dynamic_quant(x)
    out_ref = O.fused_experts_w8a8_allgather_ep(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, (0, n_local))
    sh = None
    if shared:
        out_ref = out_ref + O.shared_expert_mlp(x, *lay.shared)
        sh = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"])
    out = env.ops.moe_w8a8_layer(x.cuda(), None, w.cuda(), ids.cuda(), 0, n_local, d["w13"], d["s13"], d["w2"], d["s2"], sh,
                                 H=H, I=I)
    _check_out(out, out_ref)


# ------------------------------------------------------------------ config 4: Pangu-Ultra-MoE shape
@pytest.mark.parametrize("T", [1, 16, 128, 1024])
def test_config4_pangu_shape(env, T):
    """H=7680, I=2048, 4 local experts of 32, top-8 sigmoid grouped routing, shared expert.
    1024 tokens put both GEMMs on the tile kernel at these widths (120 k-steps, 30 column tiles)."""
    blk, lay, gate_w, bias, lo = _dsv3_block(env, 4, 8, 1, H=7680, I=2048, seed=31)
    x = tokens(T, 7680, 31 + T)
    logits = blk.gate(x.cuda().float())[0]
    out_ref, st = _block_reference(lay, x, logits.cpu(), bias, lo, 4)
    out, _ = blk(x.cuda(), None, None, 3)
    _check_out(out, out_ref, exact=True)   # fp32 rows at every size (the block's default): bit equality


# ------------------------------------------------------------------ config 5: skewed load
def test_config5_zipf_skew(env):
    """Zipf(1.2) popularity over the local experts with empty experts: 8 local experts of 64, 2 of
    them receive nothing, 512 tokens, routing by the grouped sigmoid router over biased logits."""
    n_local, E, T, H, I = 8, 64, 512, 1024, 512
    lay = Layer(n_local, H, I, seed=41)
    d = lay.to_device()
    g = gen(42)
    x = tokens(T, H, 42)
    logits = torch.randn(T, E, generator=g)
    logits[:, :n_local] += O.zipf_logit_offsets(n_local, g, 1.2, n_empty=2) + 3.0
    bias = torch.randn(E, generator=g) * 0.01
    w_ref, id_ref = O.route_noaux_tc(logits, bias, 8, 8, 4, 2.5)
    w, ids, _ = env.ops.npu_moe_gating_top_k(logits.cuda(), 8, bias.cuda(), 4, 8, 1, 0, 1, 2.5, 1e-20)
    assert torch.equal(ids.cpu(), id_ref) and torch.equal(w.cpu(), w_ref)
    counts = torch.bincount(id_ref[id_ref < n_local].long(), minlength=n_local)
    assert int((counts == 0).sum()) >= 2 and counts.max() > 3 * counts[counts > 0].float().mean() / 2
    xq, xs = O.dynamic_quant(x)
    out_ref = O.fused_experts_w8a8_allgather_ep(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w_ref, id_ref, (0, n_local))
    out = env.ops.moe_w8a8_layer(x.cuda(), None, w, ids, 0, n_local, d["w13"], d["s13"], d["w2"], d["s2"], None,
                                 H=H, I=I)
    _check_out(out, out_ref)
    # independent witness of the index logic: dense brute force in float64
    brute = O.dense_bruteforce(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w_ref, id_ref, (0, n_local))
    assert rel_err(out.float().cpu(), brute) <= REL_TOL


# ------------------------------------------------------------------ full-size properties (no oracle needed)
def _full_size_layer(env, T, seed=0):
    """32 local experts + shared at DeepSeek-V3 widths with random int8 weights made on the GPU."""
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(seed)
    H, I, n = 7168, 2048, 32
    w13 = torch.randint(-127, 128, (n + 1, 2 * I, H), generator=g, device=dev, dtype=torch.int8)
    w2 = torch.randint(-127, 128, (n + 1, H, I), generator=g, device=dev, dtype=torch.int8)
    s13 = torch.rand(n + 1, 2 * I, generator=g, device=dev) * 1e-3 + 1e-4
    s2 = torch.rand(n + 1, H, generator=g, device=dev) * 1e-3 + 1e-4
    p13, p2 = env.ops.pack_weight(w13, 1), env.ops.pack_weight(w2, 1)
    del w13, w2
    return dict(w13=p13[:n], w2=p2[:n], s13=s13[:n].contiguous(), s2=s2[:n].contiguous(), sh13=p13[n], sh2=p2[n],
                sh_s13=s13[n].contiguous(), sh_s2=s2[n].contiguous(), H=H, I=I, n=n)


@pytest.mark.parametrize("T", [64, 8192])
def test_full_size_properties(env, T):
    """At the benchmark sizes (config 2: 64 tokens, config 3: 8192 tokens, 32 local experts):
    (a) determinism: two runs give identical bits; (b) token permutation equivariance: permuting the
    tokens permutes the output rows bit for bit (the sort, the tile schedule and the combine do not
    leak order); (c) routing-weight linearity in a power of two: doubling every routing weight and
    dropping the shared expert doubles the output exactly."""
    d = _full_size_layer(env, T)
    H, I, n = d["H"], d["I"], d["n"]
    g = gen(T)
    x = tokens(T, H, 100 + T, outlier_frac=0.001 if T > 64 else 0.0).cuda()
    ids = O.local_dense_ids(T, 8, n, g).cuda()
    w = torch.rand(T, 8, generator=g).cuda()
    shared = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"])

    def run(x_, w_, ids_, sh=shared):
        return env.ops.moe_w8a8_layer(x_, None, w_, ids_, 0, n, d["w13"], d["s13"], d["w2"], d["s2"], sh, H=H, I=I)

    a = run(x, w, ids)
    b = run(x, w, ids)
    assert torch.equal(a, b), "not deterministic"
    assert bool(torch.isfinite(a.float()).all())
    perm = torch.randperm(T, generator=g).cuda()
    c = run(x[perm], w[perm], ids[perm])
    assert torch.equal(c, a[perm]), "token permutation changed the per-token results"
    e1 = run(x, w, ids, None)
    e2 = run(x, w * 2, ids, None)
    assert torch.equal(e2.float(), e1.float() * 2), "routing weights are not applied linearly"


# ------------------------------------------------------------------ HIP graph capture of the call sequence
@pytest.mark.parametrize("T", [64, 600])
def test_layer_call_sequence_is_graph_capturable(env, T):
    """Router + whole-layer entry captured in a HIP graph (no allocation, synchronisation or host read
    inside the library), replayed three times with eager work and synchronisations in between; every
    replay must give the bits of the eager run, also after the inputs changed in place.  64 tokens run
    the stream kernels; 600 tokens the tile kernel, whose few tiles share their reductions between
    blocks through counters that every launch clears with a kernel of its own."""
    K, E, n, H, I = 8, 32, 4, 1024, 512
    lay = Layer(n, H, I, seed=77, shared=True)
    d = lay.to_device()
    g = gen(78)
    x = tokens(T, H, 79).cuda()
    logits = torch.randn(T, E, generator=g).cuda()
    bias = (torch.randn(E, generator=g) * 0.01).cuda()
    ops, L = env.ops, env.L
    need = L.lib().omni_moe_w8a8_layer_workspace_bytes(T, K, n, H, I, 1, L.OMNI_DT_F32)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    out = torch.empty(T, H, dtype=torch.bfloat16, device="cuda")
    shared = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"])

    def step():
        w, ids, _ = ops.npu_moe_gating_top_k(logits, K, bias, 4, 8, 1, 0, 1, 2.5, 1e-20)
        return ops.moe_w8a8_layer(x, None, w, ids, 0, n, d["w13"], d["s13"], d["w2"], d["s2"], shared, H=H, I=I,
                                  workspace=ws, out=out)

    eager = step().clone()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                               # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        step()
    for rep in range(3):
        out.zero_()
        junk = torch.randn(256, 256, device="cuda") @ torch.randn(256, 256, device="cuda")   # eager work in between
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {rep} differs from the eager run"
        del junk
    # new inputs in the captured buffers
    x.copy_(tokens(T, H, 80).cuda())
    logits.copy_(torch.randn(T, E, generator=g).cuda())
    graph.replay()
    torch.cuda.synchronize()
    replayed = out.clone()
    assert torch.equal(step(), replayed), "replay on new inputs differs from the eager run"


# ------------------------------------------------------------------ the A2 platform branch of apply()
@pytest.mark.parametrize("shape", ["config1_toy", "config3_reduced"])
@pytest.mark.parametrize("pd_seperate_prefill", [False, True])
def test_apply_a2_platform_branch(env, monkeypatch, shape, pd_seperate_prefill):
    """``ASCEND_PLATFORM=A2`` sends the all-gather expert-parallel branch of ``apply()`` to
    ``fused_experts_w8a8_allgather_ep_a2`` (compressed_tensors_moe.py:157-170; fused_moe.py:844-937): smoothing
    factors inside the dequant-SwiGLU-quant step (other than one here, so that they show), and under
    ``pd_seperate_prefill`` the bf16 GEMM2 + finalize tail with a bf16 w2 scale.  The toy layer of config 1 as rank 1
    of 2 (stream kernels) and config 3 reduced to 2 local experts of 16 with outlier channels (tile kernels), bit
    exact against the oracle's A2 pipeline."""
    monkeypatch.setenv("ASCEND_PLATFORM", "A2")
    env.config.update_model_extra_config(enable_moe_expert_parallel=True, moe_dispatch_combine=False,
                                         prefill_dispatch_combine=False, pd_seperate_prefill=pd_seperate_prefill)
    try:
        if shape == "config1_toy":
            n_local, E, K, H, I, T, ep, rank, out_frac = 4, 8, 2, 1024, 512, 64, 2, 1, 0.0
        else:
            n_local, E, K, H, I, T, ep, rank, out_frac = 2, 16, 4, 7168, 2048, 1024, 8, 3, 0.001
        lay = _bf16_scales(Layer(n_local, H, I, seed=61))
        m = _make_fused_moe(env, lay, E, K, ep, rank)
        m.quant_method.process_weights_after_loading(m)
        assert bool((m.quant_method.smooth_scale == 1).all())          # what the reference makes (:113)
        g = gen(62)
        smooth = torch.rand(n_local, I, generator=g) * 1.5 + 0.25
        m.quant_method.smooth_scale = smooth.cuda()
        x = tokens(T, H, 63, outlier_frac=out_frac)
        lo = rank * n_local
        if shape == "config1_toy":
            ids = torch.rand(T, E, generator=g).argsort(dim=1)[:, :K].to(torch.int32)
        else:   # every token on both local experts and on two remote ones
            ids = torch.cat([(torch.rand(T, 2, generator=g).argsort(dim=1) + lo).to(torch.int32),
                             torch.randint(8, 16, (T, 2), generator=g).to(torch.int32)], dim=1)
        w = torch.rand(T, K, generator=g)
        xq, xs = O.dynamic_quant(x)
        ref = O.fused_experts_w8a8_allgather_ep_a2(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, (lo, lo + n_local),
                                                   smooth, pd_seperate_prefill=pd_seperate_prefill)
        out = m(xq.cuda(), w.cuda(), ids.cuda(), xs.cuda(), None)
        _check_out(out, ref)
        # with the factors the reference ships (ones) the branch gives the bits of the A3 pipeline
        if not pd_seperate_prefill:
            m.quant_method.smooth_scale = torch.ones(n_local, I, device="cuda")
            ref3 = O.fused_experts_w8a8_allgather_ep(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, (lo, lo + n_local))
            _check_out(m(xq.cuda(), w.cuda(), ids.cuda(), xs.cuda(), None), ref3)
    finally:
        env.config.update_model_extra_config(pd_seperate_prefill=False)
        env.dist.set_virtual_ep(1, 0)


def test_gemm1_quant_scale_on_both_kernels_and_split_k(env):
    """The smoothing factors in every GEMM1 epilogue that exists: the stream kernel that applies SwiGLU itself,
    its split-k form finished by the row kernel (forced through the tuning variable), and the tile kernel;
    int8 rows and row scales against the oracle's dequant-SwiGLU-quant with ``quant_scale``."""
    import os
    L, ops = env.L, env.ops
    G, H, I = 3, 1024, 256
    lay = Layer(G, H, I, seed=71)
    d = lay.to_device()
    g = gen(72)
    smooth = torch.rand(G, I, generator=g) * 1.5 + 0.25
    for rows_per_group, env_g1 in ((9, None), (9, "1,1,4,2"), (150, None)):
        counts = torch.tensor([rows_per_group, 0, rows_per_group + 3])
        M = int(counts.sum())
        x = tokens(M, H, 73 + rows_per_group)
        xq, xs = O.dynamic_quant(x)
        acc = O.grouped_matmul_int32(xq, lay.w1_t, counts)
        hq_ref, hs_ref = O.dequant_swiglu_quant(acc, lay.s13, xs, counts, quant_scale=smooth)
        if env_g1:
            os.environ["OMNI_MOE_G1"] = env_g1
            L.lib().omni_moe_reload_tuning()
        try:
            offsets = ops.group_offsets(counts.cuda())
            hq, hs, _ = ops.grouped_gemm1_swiglu_quant(xq.cuda(), xs.cuda(), None, 0, 1, d["w13"], d["s13"], offsets, H, I, M,
                                                       quant_scale=smooth.cuda())
            torch.cuda.synchronize()
        finally:
            if env_g1:
                del os.environ["OMNI_MOE_G1"]
                L.lib().omni_moe_reload_tuning()
        assert torch.equal(hs.cpu(), hs_ref), f"row scales, {rows_per_group} rows per group, G1={env_g1}"
        assert torch.equal(hq.cpu(), hq_ref), f"int8 rows, {rows_per_group} rows per group, G1={env_g1}"
