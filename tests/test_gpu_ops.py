"""Per-operator parity of the HIP kernels against the CPU oracle (bit exact), through the C ABI."""
import os

import pytest
import torch

from oracle import moe_oracle as O
from tests.helpers import Layer, gen, tokens

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from omni_infer_amd import hip_ops
    return hip_ops


def _eq(a, b, what):
    a, b = a.cpu(), b.cpu()
    assert a.shape == b.shape, f"{what}: shape {tuple(a.shape)} vs {tuple(b.shape)}"
    if a.dtype.is_floating_point:
        same = (a.view(torch.int32 if a.dtype == torch.float32 else torch.int16) ==
                b.view(torch.int32 if b.dtype == torch.float32 else torch.int16)) | (a == b)
    else:
        same = a == b
    bad = int((~same).sum())
    assert bad == 0, f"{what}: {bad} of {a.numel()} elements differ; first at {torch.nonzero(~same)[0].tolist()}"


# ------------------------------------------------------------------ routing
@pytest.mark.parametrize("T,E,ng,tg,K", [(1, 256, 8, 4, 8), (64, 256, 8, 4, 8), (333, 256, 8, 4, 8),
                                         (50, 64, 4, 2, 6), (17, 160, 8, 3, 6), (40, 384, 8, 4, 8)])
def test_route_noaux_tc(ops, T, E, ng, tg, K):
    g = gen(1)
    logits = torch.randn(T, E, generator=g) * 2
    bias = torch.randn(E, generator=g) * 0.01
    w_ref, id_ref = O.route_noaux_tc(logits, bias, K, ng, tg, 2.5)
    w, ids, _ = ops.npu_moe_gating_top_k(logits.cuda(), K, bias.cuda(), tg, ng, 1, 0, 1, 2.5, 1e-20)
    _eq(ids, id_ref, "ids")
    _eq(w, w_ref, "weights")


def test_route_noaux_tc_ties(ops):
    # many exactly equal logits: ties must go to the lower expert / group id
    g = gen(2)
    logits = torch.randint(-2, 3, (128, 256), generator=g).float()
    bias = torch.zeros(256)
    w_ref, id_ref = O.route_noaux_tc(logits, bias, 8, 8, 4, 2.5)
    w, ids, _ = ops.npu_moe_gating_top_k(logits.cuda(), 8, bias.cuda(), 4, 8, 1, 0, 1, 2.5, 1e-20)
    _eq(ids, id_ref, "ids")
    _eq(w, w_ref, "weights")


@pytest.mark.parametrize("scoring,with_bias", [("softmax", False), ("sigmoid", False), ("sigmoid", True)])
def test_route_grouped_topk(ops, scoring, with_bias):
    from omni_infer_amd.layers.fused_moe import grouped_topk
    g = gen(3)
    T, E = 97, 256
    logits = torch.randn(T, E, generator=g)
    bias = torch.randn(E, generator=g) * 0.01 if with_bias else None
    w_ref, id_ref, row_ref = O.route_grouped_topk(logits, 8, True, 8, 4, scoring, bias)
    w, ids, row = grouped_topk(None, logits.cuda(), 8, True, 8, 4, scoring, None if bias is None else bias.cuda())
    _eq(ids, id_ref, "ids")
    _eq(w, w_ref, "weights")
    _eq(row.contiguous(), row_ref, "row_idx")


@pytest.mark.parametrize("T,E,K,renorm", [(64, 8, 2, True), (64, 8, 2, False), (5, 64, 4, True), (33, 200, 6, True),
                                          (9, 512, 8, True)])
def test_route_softmax_topk(ops, T, E, K, renorm):
    from omni_infer_amd.layers.fused_moe import fused_topk
    logits = torch.randn(T, E, generator=gen(4)) * 3
    w_ref, id_ref, row_ref = O.route_softmax_topk(logits, K, renorm)
    w, ids, row = fused_topk(logits.cuda(), K, renorm)
    _eq(ids, id_ref, "ids")
    _eq(w, w_ref, "weights")
    _eq(row.contiguous(), row_ref, "row_idx")


# ------------------------------------------------------------------ dynamic quant
@pytest.mark.parametrize("T,H,dtype", [(64, 7168, torch.bfloat16), (3, 7680, torch.bfloat16), (5, 1024, torch.bfloat16),
                                       (7, 100, torch.bfloat16), (2, 16384, torch.bfloat16),
                                       (6, 2048, torch.float32), (4, 520, torch.float16)])
def test_dynamic_quant(ops, T, H, dtype):
    x = (torch.randn(T, H, generator=gen(5)) * 3).to(dtype)
    x[:, :: max(1, H // 7)] *= 50          # outlier channels
    if T > 1:
        x[1] = 0                             # an all-zero row
    q_ref, s_ref = O.dynamic_quant(x)
    q, s = ops.npu_dynamic_quant(x.cuda())
    _eq(s, s_ref, "scale")
    _eq(q, q_ref, "q")


def test_dynamic_quant_strided_and_3d(ops):
    x = torch.randn(4, 6, 512, generator=gen(6)).to(torch.bfloat16)
    q_ref, s_ref = O.dynamic_quant(x)
    q, s = ops.npu_dynamic_quant(x.cuda())
    _eq(q, q_ref, "q")
    _eq(s, s_ref, "scale")
    big = torch.randn(8, 1024, generator=gen(7)).to(torch.bfloat16)
    view = big[:, :512]                      # row stride 1024, 512 columns
    q_ref, s_ref = O.dynamic_quant(view)
    q, s = ops.npu_dynamic_quant(big.cuda()[:, :512])
    _eq(q, q_ref, "q strided")
    _eq(s, s_ref, "scale strided")


# ------------------------------------------------------------------ permutation
@pytest.mark.parametrize("T,K,E,lo,hi", [(64, 8, 256, 0, 32), (64, 8, 256, 96, 128), (1, 8, 256, 0, 32),
                                         (500, 8, 256, 32, 64), (2048, 8, 256, 0, 32), (700, 6, 64, 0, 64),
                                         (64, 2, 8, 0, 8), (1100, 8, 256, 0, 256),
                                         # either side of the sizes where the sort changes its block shape
                                         (100, 8, 256, 0, 32), (128, 8, 256, 0, 32), (129, 8, 256, 0, 32),
                                         (512, 8, 256, 0, 32), (513, 8, 256, 0, 32)])
def test_permute_v2(ops, T, K, E, lo, hi):
    g = gen(8)
    ids = torch.rand(T, E, generator=g).argsort(dim=1)[:, :K].to(torch.int32)
    x = torch.randint(-128, 128, (T, 64), generator=g, dtype=torch.int8)
    sc = torch.rand(T, generator=g)
    rows_ref, idx_ref, counts_ref, sc_ref = O.moe_init_routing_v2(x, ids, sc, (lo, hi))
    rows, idx, counts, scg = ops.npu_moe_init_routing_v2(x.cuda(), ids.cuda(), scale=sc.cuda(),
                                                         active_expert_range=[lo, hi], expert_num=E)
    m = idx_ref.numel()
    _eq(counts, counts_ref, "counts")
    _eq(idx[:m], idx_ref, "expanded_x_idx")
    _eq(rows[:m], rows_ref, "rows")
    _eq(scg[:m], sc_ref, "scale")
    # the tail holds the dropped assignments in their original order: still a permutation
    assert sorted(idx.cpu().tolist()) == list(range(T * K))


def test_permute_v1_and_empty(ops):
    g = gen(9)
    T, K, E = 200, 2, 8
    ids = torch.rand(T, E, generator=g).argsort(dim=1)[:, :K].to(torch.int32)
    ids[ids == 3] = 5                        # expert 3 receives nothing (and 5 may repeat in a token)
    x = torch.randn(T, 32, generator=g).to(torch.bfloat16)
    row_idx = torch.arange(T * K, dtype=torch.int32).view(K, T).t().contiguous()
    rows_ref, s2d_ref, sid_ref = O.moe_init_routing_v1(x, row_idx, ids)
    rows, s2d, sid = ops.npu_moe_init_routing(x.cuda(), row_idx.cuda(), ids.cuda(), T, num_experts=E)
    _eq(rows, rows_ref, "rows")
    _eq(s2d, s2d_ref, "src_to_dst")
    _eq(sid, sid_ref, "sorted ids")
    cum = ops.npu_moe_compute_expert_tokens(sid, E)
    _eq(cum, O.compute_expert_tokens(sid_ref, E).to(torch.int32), "cumulative tokens")


def test_permute_all_dropped(ops):
    ids = torch.full((16, 4), 200, dtype=torch.int32)
    from omni_infer_amd import _lib as L
    p = ops.moe_permute(ids.cuda(), 0, 32, L.OMNI_IDX_TOKEN_MAJOR)
    assert int(p.counts.sum()) == 0 and int(p.offsets[-1]) == 0
    assert bool((p.src_to_dst.cpu() == -1).all())


# ------------------------------------------------------------------ weight packing
@pytest.mark.parametrize("layout", [0, 1])
def test_pack_weight_layout(ops, layout):
    g = gen(10)
    G, Kd, N = 2, 128, 48
    w = torch.randint(-128, 128, (G, Kd, N), generator=g, dtype=torch.int8)      # logical [G, K, N]
    src = w if layout == 0 else w.transpose(1, 2).contiguous()
    packed = ops.pack_weight(src.cuda(), layout).cpu().view(G, -1)
    k = torch.arange(Kd).view(-1, 1)
    n = torch.arange(N).view(1, -1)
    off = (((n // 16) * (Kd // 64) + k // 64) * 64 + (n % 16) + 16 * ((k % 64) // 16)) * 16 + k % 16
    for gi in range(G):
        assert bool((packed[gi][off.reshape(-1)] == w[gi].reshape(-1)).all())


# ------------------------------------------------------------------ GEMM1 / GEMM2 / combine
def _grouped_case(T, K, n_local, E, H, I, seed, lo=0):
    g = gen(seed)
    lay = Layer(n_local, H, I, seed)
    x = tokens(T, H, seed + 1)
    xq, xs = O.dynamic_quant(x)
    ids = torch.rand(T, E, generator=g).argsort(dim=1)[:, :K].to(torch.int32)
    w = torch.rand(T, K, generator=g)
    return lay, xq, xs, ids, w


@pytest.mark.parametrize("T,K,n_local,E,H,I,force", [
    (64, 2, 8, 8, 1024, 512, 0),        # toy shape, stream kernel
    (64, 8, 4, 32, 7168, 2048, 0),      # DeepSeek-V3 widths, 4 local experts of 32
    (16, 8, 4, 32, 7680, 2048, 0),      # Pangu widths
    (300, 4, 4, 8, 1024, 512, 1),       # ragged groups > 64 rows through the stream kernel
    (300, 4, 4, 8, 1024, 512, 2),       # same through the tile kernel
    (1100, 4, 3, 6, 512, 256, 0),       # tile kernel by default, partial 256-row blocks
    (700, 2, 3, 3, 1024, 512, 2),       # tile kernel, 24 tiles per GEMM: each tile's reduction is shared by four blocks
    (520, 1, 1, 1, 2048, 1024, 2),      # one group of three row blocks: 24 / 96 tiles, split four ways / two ways
])
def test_gemm1_gemm2_stages(ops, T, K, n_local, E, H, I, force, tuning):
    from omni_infer_amd import _lib as L
    if force:
        tuning(OMNI_MOE_FORCE_KERNEL=force)
        want = {1: "gemm_stream", 2: "gemm_pipe"}[force]
        for kind in (1, 2):   # the forced kernel is the one the library will launch
            assert ops.gemm_kernel_name(kind, T, K, n_local, 0, T * K, H, I).startswith(want)
    lay, xq, xs, ids, w = _grouped_case(T, K, n_local, E, H, I, 20 + T)
    d = lay.to_device()
    out_ref, st = O.fused_experts_w8a8_allgather_ep(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, (0, n_local),
                                                    return_stages=True)
    p = ops.moe_permute(ids.cuda(), 0, n_local, L.OMNI_IDX_TOKEN_MAJOR)
    m = int(st["counts"].sum())
    M_cap = T * K
    h_q, h_s, acc1 = ops.grouped_gemm1_swiglu_quant(xq.cuda(), xs.cuda(), p.sorted_src, L.OMNI_IDX_TOKEN_MAJOR, K,
                                                    d["w13"], d["s13"], p.offsets, H, I, M_cap, want_acc=True)
    _eq(acc1[:m], st["acc1"], "GEMM1 int32 accumulators")
    _eq(h_s[:m], st["h_s"], "stage-2 scales")
    _eq(h_q[:m], st["h_q"], "stage-2 int8 activations")
    # without the accumulator dump the small-batch kernel applies SwiGLU itself: same bits
    h_q2, h_s2, _ = ops.grouped_gemm1_swiglu_quant(xq.cuda(), xs.cuda(), p.sorted_src, L.OMNI_IDX_TOKEN_MAJOR, K,
                                                   d["w13"], d["s13"], p.offsets, H, I, M_cap)
    _eq(h_s2[:m], st["h_s"], "stage-2 scales (no dump)")
    _eq(h_q2[:m], st["h_q"], "stage-2 int8 activations (no dump)")
    for dt in (torch.float32, torch.bfloat16):
        rows, acc2 = ops.grouped_gemm2_dequant(h_q, h_s, d["w2"], d["s2"], p.offsets, H, I, out_dtype=dt, want_acc=True)
        _eq(acc2[:m], st["acc2"], "GEMM2 int32 accumulators")
        g_of = torch.repeat_interleave(torch.arange(n_local), st["counts"])
        ref_rows = ((st["acc2"].float() * lay.s2[g_of]) * st["h_s"].unsqueeze(-1)).to(dt)
        _eq(rows[:m], ref_rows, f"GEMM2 rows {dt}")
    rows32, _ = ops.grouped_gemm2_dequant(h_q, h_s, d["w2"], d["s2"], p.offsets, H, I, out_dtype=torch.float32)
    out = ops.moe_combine(rows32, w.cuda(), p.src_to_dst, L.OMNI_IDX_TOKEN_MAJOR, L.OMNI_ORDER_SLOT)
    _eq(out, out_ref, "combined output")


def test_split_tiles_equal_unsplit(ops, tuning):
    """Tiles of the last partial round share their reduction between blocks (integer partial sums, the
    last block to arrive adds them): the results are the same bits as with the sharing switched off."""
    from omni_infer_amd import _lib as L
    T, K, n_local, E, H, I = 700, 2, 3, 3, 1024, 512
    lay, xq, xs, ids, w = _grouped_case(T, K, n_local, E, H, I, 77)
    d = lay.to_device()
    p = ops.moe_permute(ids.cuda(), 0, n_local, L.OMNI_IDX_TOKEN_MAJOR)
    got = {}
    for tail in ("1", "0"):
        tuning(OMNI_MOE_FORCE_KERNEL=2, OMNI_MOE_TILE_TAIL=tail)
        for rep in range(10):   # repeated launches reuse the same scratch and counters
            h_q, h_s, acc1 = ops.grouped_gemm1_swiglu_quant(xq.cuda(), xs.cuda(), p.sorted_src, L.OMNI_IDX_TOKEN_MAJOR, K,
                                                            d["w13"], d["s13"], p.offsets, H, I, T * K, want_acc=True)
            rows, acc2 = ops.grouped_gemm2_dequant(h_q, h_s, d["w2"], d["s2"], p.offsets, H, I,
                                                   out_dtype=torch.bfloat16, want_acc=True)
            cur = [t.cpu() for t in (h_q, h_s, acc1, rows, acc2)]
            if tail in got:
                for a, b in zip(cur, got[tail]):
                    assert torch.equal(a, b), "launches of the same call differ"
            got[tail] = cur
    for a, b, what in zip(got["1"], got["0"], ("h_q", "h_s", "acc1", "rows", "acc2")):
        m = int(p.offsets[-1])
        assert torch.equal(a[:m], b[:m]), f"{what}: split and unsplit tiles differ"


def _tile_outputs(ops, lay_dev, xq, xs, p, K, H, I, M_cap):
    from omni_infer_amd import _lib as L
    h_q, h_s, acc1 = ops.grouped_gemm1_swiglu_quant(xq, xs, p.sorted_src, L.OMNI_IDX_TOKEN_MAJOR, K, lay_dev["w13"],
                                                    lay_dev["s13"], p.offsets, H, I, M_cap, want_acc=True)
    out = [h_q, h_s, acc1]
    for dt in (torch.float32, torch.bfloat16):
        rows, acc2 = ops.grouped_gemm2_dequant(h_q, h_s, lay_dev["w2"], lay_dev["s2"], p.offsets, H, I, out_dtype=dt,
                                               want_acc=True)
        out += [rows, acc2]
    return [t.cpu() for t in out]


@pytest.mark.parametrize("T,K,n_local,E,H,I", [
    (700, 2, 3, 3, 1024, 512),     # a few row blocks per group, partial last blocks, split tiles
    (1500, 4, 6, 8, 1536, 768),    # light (at most 96 rows) and heavy last blocks mixed, reduction of 12 and 6 super-steps
    (900, 2, 2, 2, 256, 128),      # the shortest reductions: two super-steps and one
    (2100, 1, 1, 1, 384, 640),     # one group of nine row blocks; three and five super-steps (loop remainders of 0, 2 and 4 k-steps)
])
def test_tile_layouts_give_the_same_bits(ops, tuning, T, K, n_local, E, H, I):
    """The tile kernel has two layouts of the activation operand in LDS (whole 128-byte lines with the pinned
    k loop, the default where it applies, and 16-row fragments), two forms of the matrix instruction in the line
    layout (16x16x64, the default, and 32x32x32) and two tile widths: all of them give the bits of the oracle."""
    from omni_infer_amd import _lib as L
    lay, xq, xs, ids, w = _grouped_case(T, K, n_local, E, H, I, 300 + T)
    d = lay.to_device()
    _, st = O.fused_experts_w8a8_allgather_ep(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, (0, n_local),
                                              return_stages=True)
    m = int(st["counts"].sum())
    p = ops.moe_permute(ids.cuda(), 0, n_local, L.OMNI_IDX_TOKEN_MAJOR)
    M_cap = T * K
    seen = {}
    for tag, env in (("lines", dict(OMNI_MOE_TILE_LINES=1, OMNI_MOE_TILE_WN=4, OMNI_MOE_TILE_MFMA16=1)),
                     ("lines32", dict(OMNI_MOE_TILE_LINES=1, OMNI_MOE_TILE_WN=4, OMNI_MOE_TILE_MFMA16=0)),
                     ("frags", dict(OMNI_MOE_TILE_LINES=0, OMNI_MOE_TILE_WN=4)),
                     ("narrow", dict(OMNI_MOE_TILE_LINES=1, OMNI_MOE_TILE_WN=2))):
        tuning(OMNI_MOE_FORCE_KERNEL=2, **env)
        name = ops.gemm_kernel_name(1, T, K, n_local, 0, M_cap, H, I)
        assert name == {"lines": "gemm_pipe<1,4,lines>", "lines32": "gemm_pipe<1,4,lines>", "frags": "gemm_pipe<1,4,frags>",
                        "narrow": "gemm_pipe<1,2,frags>"}[tag]
        seen[tag] = _tile_outputs(ops, d, xq.cuda(), xs.cuda(), p, K, H, I, M_cap)
    h_q, h_s, acc1 = seen["lines"][:3]
    _eq(acc1[:m], st["acc1"], "GEMM1 int32 accumulators")
    _eq(h_s[:m], st["h_s"], "stage-2 scales")
    _eq(h_q[:m], st["h_q"], "stage-2 int8 activations")
    _eq(seen["lines"][4][:m], st["acc2"], "GEMM2 int32 accumulators")
    for tag in ("lines32", "frags", "narrow"):
        for a, b, what in zip(seen[tag], seen["lines"], ("h_q", "h_s", "acc1", "rows f32", "acc2", "rows bf16", "acc2")):
            assert torch.equal(a[:m], b[:m]), f"{what}: {tag} differs from the line layout"


def test_tile_kernel_odd_number_of_k_steps(ops, tuning):
    """A reduction length that is a multiple of 64 but not of 128 (17 k-steps) takes the fragment layout of the
    tile kernel; GEMM2 of this shape (1088 channels: no whole tile) goes to the stream kernel."""
    from omni_infer_amd import _lib as L
    T, K, n_local, E, H, I = 600, 2, 3, 3, 1088, 512
    tuning(OMNI_MOE_FORCE_KERNEL=2)
    assert ops.gemm_kernel_name(1, T, K, n_local, 0, T * K, H, I) == "gemm_pipe<1,4,frags>"
    lay, xq, xs, ids, w = _grouped_case(T, K, n_local, E, H, I, 411)
    d = lay.to_device()
    out_ref, st = O.fused_experts_w8a8_allgather_ep(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, (0, n_local),
                                                    return_stages=True)
    m = int(st["counts"].sum())
    p = ops.moe_permute(ids.cuda(), 0, n_local, L.OMNI_IDX_TOKEN_MAJOR)
    got = _tile_outputs(ops, d, xq.cuda(), xs.cuda(), p, K, H, I, T * K)
    _eq(got[2][:m], st["acc1"], "GEMM1 int32 accumulators")
    _eq(got[0][:m], st["h_q"], "stage-2 int8 activations")
    _eq(got[4][:m], st["acc2"], "GEMM2 int32 accumulators")
    out = ops.moe_combine(got[3].cuda(), w.cuda(), p.src_to_dst, L.OMNI_IDX_TOKEN_MAJOR, L.OMNI_ORDER_SLOT)
    _eq(out, out_ref, "combined output")


def test_combine_k_order_with_skip(ops):
    from omni_infer_amd import _lib as L
    g = gen(30)
    T, K, H, E = 50, 4, 256, 8
    ids = torch.rand(T, E, generator=g).argsort(dim=1)[:, :K].to(torch.int32)
    w = torch.rand(T, K, generator=g)
    rows = torch.randn(T * K, H, generator=g).to(torch.bfloat16)
    skip = torch.randn(T, H, generator=g).to(torch.bfloat16)
    for mode, omode in ((0, L.OMNI_IDX_K_MAJOR), (2, L.OMNI_IDX_TOKEN_MAJOR)):
        p = ops.moe_permute(ids.cuda(), 0, 6, omode)       # experts 6, 7 are not local: dropped rows
        ref = O.moe_finalize_routing(rows.float(), skip, w, p.src_to_dst.cpu(), drop_pad_mode=mode).to(torch.bfloat16)
        out = ops.moe_combine(rows.cuda(), w.cuda(), p.src_to_dst, omode, L.OMNI_ORDER_K, init=skip.cuda())
        _eq(out, ref, f"finalize mode {mode}")


# ------------------------------------------------------------------ layer entry: extreme routings and sizes
@pytest.mark.parametrize("T,K,n_local,E,pattern", [
    (200, 1, 1, 4, "first_k"),    # every token to the single local expert: 200 rows in one group (tile kernel)
    (129, 2, 4, 4, "first_k"),    # 129 rows in two groups: first size past the stream/tile switch; two empty groups
    (128, 2, 4, 4, "first_k"),    # 128 rows: last size of the stream kernel, 4 or 8 row blocks per group
    (257, 1, 2, 2, "first_k"),    # one row past a whole 256-row tile, one empty group
    (40, 4, 4, 8, "none"),        # no assignment is local: only the shared expert contributes
    (1, 8, 8, 8, "first_k"),      # one token to every expert: eight one-row groups
    (96, 3, 5, 5, "random"),      # odd group count, ragged groups
])
def test_layer_entry_extreme_routings(ops, T, K, n_local, E, pattern):
    """omni_moe_w8a8_layer (sort, both GEMMs, combine, shared expert) on routings that stress the row-block
    logic: every token on the same experts, empty groups, nothing local, boundary row counts."""
    H, I = 512, 256
    g = gen(900 + T)
    lay = Layer(n_local, H, I, seed=900 + T, shared=True)
    x = tokens(T, H, 901 + T)
    w = torch.rand(T, K, generator=g)
    if pattern == "first_k":
        ids = torch.arange(K, dtype=torch.int32).repeat(T, 1)
    elif pattern == "none":
        ids = torch.stack([torch.randperm(E - n_local, generator=g)[:K] + n_local for _ in range(T)]).to(torch.int32)
    else:
        ids = torch.rand(T, E, generator=g).argsort(dim=1)[:, :K].to(torch.int32)
    xq, xs = O.dynamic_quant(x)
    routed = O.fused_experts_w8a8_allgather_ep(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, (0, n_local))
    shared = O.shared_expert_mlp(x, *lay.shared)
    want = (routed.float() + shared.float()).to(torch.bfloat16)
    d = lay.to_device()
    out = ops.moe_w8a8_layer(x.cuda(), None, w.cuda(), ids.cuda(), 0, n_local, d["w13"], d["s13"], d["w2"], d["s2"],
                             (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"]), H=H, I=I)
    _eq(out, want, f"layer output ({pattern})")


def test_layer_entry_zero_tokens(ops):
    lay = Layer(2, 512, 256, seed=3, shared=True)
    d = lay.to_device()
    x = torch.zeros(0, 512, dtype=torch.bfloat16).cuda()
    out = ops.moe_w8a8_layer(x, None, torch.zeros(0, 2).cuda(), torch.zeros(0, 2, dtype=torch.int32).cuda(), 0, 2,
                             d["w13"], d["s13"], d["w2"], d["s2"], (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"]),
                             H=512, I=256)
    assert out.shape == (0, 512)


# ------------------------------------------------------------------ seeded sweep over small shapes
def _sweep_cases():
    """40 seeded shapes: token counts around the kernel-switch points, odd expert counts, all the
    width granularities the kernels accept (reduction lengths in multiples of 256 for the stream
    kernel, of 64 for the tile kernel), with and without the shared expert, both index modes."""
    g = gen(4242)
    cases = []
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    for n in range(40):
        E = r(1, 12)
        n_local = r(1, E)
        K = r(1, min(E, 4))
        T = [1, 2, 7, 31, 64, 65, 130, 200, 300, 513][n % 10]
        H = 256 * r(1, 3) if n % 3 else 64 * r(1, 9)
        I = 256 * r(1, 2) if n % 3 else 64 * r(1, 5)
        cases.append((T, K, n_local, E, H, I, bool(n & 1), n))
    return cases


@pytest.mark.parametrize("T,K,n_local,E,H,I,shared,seed", _sweep_cases())
def test_layer_entry_shape_sweep(ops, T, K, n_local, E, H, I, shared, seed):
    g = gen(5000 + seed)
    lay = Layer(n_local, H, I, seed=5000 + seed, shared=shared)
    x = tokens(T, H, 6000 + seed)
    ids = torch.rand(T, E, generator=g).argsort(dim=1)[:, :K].to(torch.int32)
    w = torch.rand(T, K, generator=g)
    lo = int(torch.randint(0, E - n_local + 1, (1,), generator=g))     # the local range anywhere in [0, E)
    xq, xs = O.dynamic_quant(x)
    routed = O.fused_experts_w8a8_allgather_ep(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, (lo, lo + n_local))
    want = routed
    if shared:
        want = (routed.float() + O.shared_expert_mlp(x, *lay.shared).float()).to(torch.bfloat16)
    d = lay.to_device()
    sh = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"]) if shared else None
    try:
        out = ops.moe_w8a8_layer(x.cuda(), None, w.cuda(), ids.cuda(), lo, lo + n_local, d["w13"], d["s13"], d["w2"],
                                 d["s2"], sh, H=H, I=I)
    except RuntimeError as e:
        # the only widths refused: GEMM2 can use neither kernel (stream: I % 256 == 0; tile: H % 128 == 0)
        assert I % 256 != 0 and H % 128 != 0, f"refused a supported shape: {e}"
        assert "multiple of 256" in str(e) or "not divisible" in str(e), str(e)
        return
    _eq(out, want, f"layer output T={T} K={K} n_local={n_local}/{E} H={H} I={I} shared={shared}")


# ------------------------------------------------------------------ seeded sweep over tile-kernel shapes
def _tile_sweep_cases():
    """14 seeded shapes that the 256 x 256 tile kernel with the line layout serves: hundreds to thousands of
    tokens, skewed routing (full, heavy, light and empty row blocks side by side), widths whose reductions
    are 1 to 6 super-steps of 128, with and without the shared expert."""
    g = gen(777)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    cases = []
    for n in range(14):
        E = r(1, 10)
        n_local = r(1, E)
        K = r(1, min(E, 3))
        T = [600, 900, 1300, 2200, 3100, 777, 1025][n % 7]
        cases.append((T, K, n_local, E, 256 * r(1, 3), 128 * r(1, 3), bool(n & 1), n))
    return cases


@pytest.mark.parametrize("T,K,n_local,E,H,I,shared,seed", _tile_sweep_cases())
def test_layer_entry_tile_sweep(ops, tuning, T, K, n_local, E, H, I, shared, seed):
    tuning(OMNI_MOE_FORCE_KERNEL=2)
    assert ops.gemm_kernel_name(1, T, K, n_local, T if shared else 0, T * K + (T if shared else 0), H, I) == "gemm_pipe<1,4,lines>"
    assert ops.gemm_kernel_name(2, T, K, n_local, T if shared else 0, T * K + (T if shared else 0), H, I) == "gemm_pipe<2,4,lines>"
    g = gen(7000 + seed)
    lay = Layer(n_local, H, I, seed=7000 + seed, shared=shared)
    x = tokens(T, H, 8000 + seed)
    pop = torch.randn(E, generator=g) * 1.5          # a few popular experts, a few nearly empty ones
    ids = (torch.rand(T, E, generator=g) + pop * 0.4).argsort(dim=1, descending=True)[:, :K].to(torch.int32)
    w = torch.rand(T, K, generator=g)
    lo = int(torch.randint(0, E - n_local + 1, (1,), generator=g))
    xq, xs = O.dynamic_quant(x)
    want = O.fused_experts_w8a8_allgather_ep(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, (lo, lo + n_local))
    if shared:
        want = (want.float() + O.shared_expert_mlp(x, *lay.shared).float()).to(torch.bfloat16)
    d = lay.to_device()
    sh = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"]) if shared else None
    out = ops.moe_w8a8_layer(x.cuda(), None, w.cuda(), ids.cuda(), lo, lo + n_local, d["w13"], d["s13"], d["w2"], d["s2"],
                             sh, H=H, I=I)
    _eq(out, want, f"layer output T={T} K={K} n_local={n_local}/{E} H={H} I={I} shared={shared}")


@pytest.mark.parametrize("shared", [False, True])
def test_tile_numbering_row_count_edges(ops, tuning, shared):
    """Groups whose row counts sit on every edge of the tile numbering: empty, one row, 96 and 97 rows (light /
    heavy last block), one full block, one full block plus a few rows (the small block that stays next to its
    full one), plus 96 and 97, two and more full blocks with and without a light tail."""
    tuning(OMNI_MOE_FORCE_KERNEL=2)
    counts = [0, 1, 96, 97, 256, 257, 300, 352, 353, 512, 513, 608, 609, 0, 768 + 40, 255]
    n_local, H, I = len(counts), 256, 128
    E = n_local + 3
    T = sum(counts) + 50                              # 50 tokens go to experts of other ranks
    g = gen(4242)
    ids = torch.cat([torch.full((c,), e + 2, dtype=torch.int32) for e, c in enumerate(counts)] +
                    [torch.full((25,), 0, dtype=torch.int32), torch.full((25,), E - 1, dtype=torch.int32)])
    ids = ids[torch.randperm(T, generator=g)].view(T, 1)
    w = torch.rand(T, 1, generator=g)
    lay = Layer(n_local, H, I, seed=4242, shared=shared)
    x = tokens(T, H, 4243)
    xq, xs = O.dynamic_quant(x)
    want = O.fused_experts_w8a8_allgather_ep(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w, ids, (2, 2 + n_local))
    if shared:
        want = (want.float() + O.shared_expert_mlp(x, *lay.shared).float()).to(torch.bfloat16)
    d = lay.to_device()
    sh = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"]) if shared else None
    out = ops.moe_w8a8_layer(x.cuda(), None, w.cuda(), ids.cuda(), 2, 2 + n_local, d["w13"], d["s13"], d["w2"], d["s2"],
                             sh, H=H, I=I)
    _eq(out, want, f"row-count edges shared={shared}")


@pytest.mark.parametrize("G", [1, 33, 64, 65, 200, 256])
@pytest.mark.parametrize("dtype", [torch.int32, torch.int64])
def test_group_offsets(G, dtype):
    """Row offsets of the groups from their sizes (what the reference's grouped operators make of ``group_list``
    with ``group_list_type=1``): against numpy's cumulative sum, empty groups included."""
    import numpy as np
    from omni_infer_amd import hip_ops as ops
    g = torch.Generator().manual_seed(900 + G)
    counts = torch.randint(0, 5000, (G,), generator=g).to(dtype)
    counts[torch.rand(G, generator=g) < 0.2] = 0
    off = ops.group_offsets(counts.cuda()).cpu()
    assert off.dtype == torch.int32 and off.numel() == G + 1
    assert off.tolist() == [0] + np.cumsum(counts.numpy()).tolist()
    with pytest.raises(RuntimeError, match="groups"):
        ops.group_offsets(torch.zeros(257, dtype=torch.int32, device="cuda"))
