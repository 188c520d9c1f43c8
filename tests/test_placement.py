"""Expert placement on the MoE path: the oracle against hand-worked cases, invariants and the closed form; the
library's host tables, the two device operations and the block with a redundant placement against the oracle.

Known answers taken from the reference's own tests are marked with their file and line
(omni/accelerators/placement/tests/...)."""
import os
import types

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from oracle import placement_oracle as P
from tests.helpers import Layer, gen, tokens

HERE = os.path.dirname(os.path.abspath(__file__))


def _fixture_patterns():
    z = np.load(os.path.join(HERE, "golden", "placement_patterns.npz"), allow_pickle=False)
    out = {}
    for key in z.files:
        if key.endswith("_bits"):
            name = key[:-5]
            shape = tuple(int(v) for v in z[name + "_shape"])
            out[name] = np.unpackbits(z[key])[:int(np.prod(shape))].reshape(shape).astype(np.int32)
    return out


def _random_pattern(rng, world, layers, experts, extra_per_device):
    """Base placement (expert e on device e // (experts // world)) plus `extra_per_device` random copies each."""
    per = experts // world
    pat = np.zeros((world, layers, experts), dtype=np.int32)
    for r in range(world):
        pat[r, :, r * per:(r + 1) * per] = 1
        for layer in range(layers):
            others = np.setdiff1d(np.arange(experts), np.arange(r * per, (r + 1) * per))
            n_extra = int(rng.integers(0, extra_per_device + 1))
            pat[r, layer, rng.choice(others, size=n_extra, replace=False)] = 1
    return pat


def _num_deploy(pat):
    world = pat.shape[0]
    return max(int(pat.sum(axis=(0, 2)).max()) // world, int(pat.sum(axis=2).max()), 1) * world


def _closed_form_selector(pat, num_deploy, rank, devices_per_host):
    """The rule in one sentence, written without the reference's scan: take the copy on the rank itself, else the
    (rank mod n)-th of the n copies on the rank's host, else the (rank mod m)-th of the m other copies, copies in
    ascending position order."""
    world, layers, experts = pat.shape
    per = num_deploy // world
    sel = np.zeros((layers, experts), dtype=np.int32)
    for layer in range(layers):
        start = {}
        for r in range(world):
            for i, e in enumerate(np.nonzero(pat[r, layer])[0]):
                start.setdefault(int(e), []).append(r * per + i)
        for e, positions in start.items():
            positions = sorted(positions)
            own = [p for p in positions if p // per == rank]
            same = [p for p in positions if p // per != rank and (p // per) // devices_per_host == rank // devices_per_host]
            far = [p for p in positions if (p // per) // devices_per_host != rank // devices_per_host]
            sel[layer, e] = own[0] if own else (same[rank % len(same)] if same else far[rank % len(far)])
    return sel


# ------------------------------------------------------------------------------------------ oracle pins (CPU)
HAND = np.zeros((4, 1, 4), dtype=np.int32)
for _dev, _experts in enumerate([(0, 1), (2, 3), (0, 2), (1, 3)]):
    HAND[_dev, 0, list(_experts)] = 1


def test_oracle_tables_hand_worked_cases():
    """4 devices x 2 positions; device d deploys: 0:{0,1} 1:{2,3} 2:{0,2} 3:{1,3}.  Positions follow by hand:
    [e0 e1 | e2 e3 | e0 e2 | e1 e3]."""
    assert P.position_table(HAND, 8).tolist() == [[0, 1, 2, 3, 0, 2, 1, 3]]
    # two devices per host: rank 0 has e0, e1 itself and finds e2, e3 on its host neighbour (positions 2, 3)
    assert P.selector_table(HAND, 8, 0, 2).tolist() == [[0, 1, 2, 3]]
    # rank 2 (host 1): own e0 at 4, e2 at 5; e1 and e3 on device 3 of its host
    assert P.selector_table(HAND, 8, 2, 2).tolist() == [[4, 6, 5, 7]]
    # every device its own host: all foreign copies are distant, shared out by rank mod 2
    assert P.selector_table(HAND, 8, 1, 1).tolist() == [[4, 6, 2, 3]]   # e0: [0,4][1], e1: [1,6][1]
    assert P.selector_table(HAND, 8, 3, 1).tolist() == [[4, 6, 5, 7]]   # e0: [0,4][1], e2: [2,5][1]
    assert P.selector_table(HAND, 8, 0, 1).tolist() == [[0, 1, 2, 3]]   # e2: [2,5][0], e3: [3,7][0]
    # one host of four: foreign copies are same-host candidates
    assert P.selector_table(HAND, 8, 3, 4).tolist() == [[4, 6, 5, 7]]   # e0: [0,4][3%2], e2: [2,5][3%2]
    assert P.selector_table(HAND, 8, 2, 4).tolist() == [[4, 1, 5, 3]]   # e1: [1,6][0], e3: [3,7][0]
    # a single copy is taken wherever it is; unused positions stay -1
    single = np.zeros((2, 1, 3), dtype=np.int32)
    single[0, 0, [0, 1]] = 1
    single[1, 0, [2]] = 1
    assert P.position_table(single, 4).tolist() == [[0, 1, 2, -1]]
    assert P.selector_table(single, 4, 0, 1).tolist() == [[0, 1, 2]]
    assert P.selector_table(single, 4, 1, 1).tolist() == [[0, 1, 2]]


@pytest.mark.parametrize("seed", range(6))
def test_oracle_selector_against_closed_form_and_invariants(seed):
    rng = np.random.default_rng(seed)
    world = int(rng.choice([2, 4, 8, 16]))
    experts = world * int(rng.choice([2, 4, 8]))
    dph = int(rng.choice([1, 2, 4, 8]))
    pat = _random_pattern(rng, world, 3, experts, 3)
    nd = _num_deploy(pat)
    per = nd // world
    pos = P.position_table(pat, nd)
    for rank in range(world):
        sel = P.selector_table(pat, nd, rank, dph)
        assert np.array_equal(sel, _closed_form_selector(pat, nd, rank, dph))
        for layer in range(3):
            chosen = pos[layer][sel[layer]]
            assert np.array_equal(chosen, np.arange(experts))            # every position holds the expert asked for
            mine = pat[rank, layer] == 1
            assert np.all(sel[layer][mine] // per == rank)               # an own copy always wins
    # position table: a device's experts in ascending id, then -1
    for layer in range(3):
        for r in range(world):
            row = pos[layer, r * per:(r + 1) * per]
            want = np.nonzero(pat[r, layer])[0]
            assert np.array_equal(row[:len(want)], want) and np.all(row[len(want):] == -1)


def test_oracle_selector_on_the_reference_patterns():
    """Slices of the placement patterns the reference's placement tests hold as data."""
    for name, pat in _fixture_patterns().items():
        world, layers, experts = pat.shape
        nd = max(int(pat.sum(axis=(0, 2)).max()) // world, 1) * world   # expert_mapping.py:33
        per = nd // world
        assert int(pat.sum(axis=2).max()) <= per, name
        pos = P.position_table(pat, nd)
        copies = pat.sum(axis=0)
        for rank in (0, 1, world // 2, world - 1):
            for dph in (8, 16):
                sel = P.selector_table(pat, nd, rank, dph)
                assert np.array_equal(sel, _closed_form_selector(pat, nd, rank, dph)), name
                for layer in range(layers):
                    assert np.array_equal(pos[layer][sel[layer]], np.arange(experts)), name
                    # a copy on the rank's host wins over a distant one
                    host_of = (sel[layer] // per) // dph
                    for e in np.nonzero(copies[layer] > 1)[0]:
                        on_host = [r for r in np.nonzero(pat[:, layer, e])[0] if r // dph == rank // dph]
                        if on_host:
                            assert host_of[e] == rank // dph, (name, layer, e)
        # the ranks of one host spread over the same-host copies of an expert none of them deploys
        dph = 8
        for layer in range(layers):
            for e in np.nonzero(copies[layer] > 1)[0][:16]:
                holders = np.nonzero(pat[:, layer, e])[0]
                for host in range(world // dph):
                    on_host = [r for r in holders if r // dph == host]
                    asking = [r for r in range(host * dph, (host + 1) * dph) if r not in on_host]
                    if len(on_host) < 2 or not asking:
                        continue
                    got = {int(P.selector_table(pat[:, layer:layer + 1], nd, r, dph)[0, e]) for r in asking}
                    assert len(got) == min(len(on_host), len({r % len(on_host) for r in asking})), (name, layer, e)


def test_oracle_remap_and_counters():
    g = gen(5)
    table = torch.randperm(40, generator=g)[:32].to(torch.int32)
    ids = torch.randint(0, 32, (17, 8), generator=g)
    want = torch.nn.functional.embedding(ids, table.unsqueeze(-1).long()).squeeze(-1)   # the reference's call
    assert np.array_equal(P.remap_ids(ids.numpy(), table.unsqueeze(-1).numpy()), want.numpy())
    counts = np.array([0, 5, 10**16 - 3, 10**16 - 1], dtype=np.int64)
    add = np.array([7, 0, 2, 9], dtype=np.int32)
    got = P.record_activation(counts, add, 10**16)
    assert got.tolist() == [(int(c) + int(a)) % 10**16 for c, a in zip(counts, add)] == [7, 5, 10**16 - 1, 8]


# ------------------------------------------------------------------------------------------ host tables (CPU)
def test_library_tables_against_oracle():
    from omni_infer_amd import hip_ops as ops
    rng = np.random.default_rng(11)
    cases = [(HAND, 8, 2)]
    for _ in range(4):
        world = int(rng.choice([2, 4, 8]))
        cases.append((_random_pattern(rng, world, 2, world * 4, 2), None, int(rng.choice([1, 2, 4]))))
    for name, pat in _fixture_patterns().items():
        cases.append((pat, max(int(pat.sum(axis=(0, 2)).max()) // pat.shape[0], 1) * pat.shape[0], 8))
    for pat, nd, dph in cases:
        nd = nd or _num_deploy(pat)
        for rank in sorted({0, pat.shape[0] // 2, pat.shape[0] - 1}):
            pos, sel = ops.placement_tables(torch.from_numpy(pat), rank, dph, nd)
            assert np.array_equal(pos.numpy(), P.position_table(pat, nd))
            assert np.array_equal(sel.numpy(), P.selector_table(pat, nd, rank, dph))


def test_library_tables_reject_bad_patterns():
    from omni_infer_amd import hip_ops as ops
    bad = torch.from_numpy(HAND.copy())
    bad[0, 0, 0] = 2
    with pytest.raises(ValueError):
        ops.placement_tables(bad, 0, 2, 8)
    with pytest.raises(ValueError):
        ops.placement_tables(torch.from_numpy(HAND), 4, 2, 8)       # rank outside the pattern
    with pytest.raises(ValueError):
        ops.placement_tables(torch.from_numpy(HAND), 0, 2, 4)       # 2 experts per device do not fit 1 position
    with pytest.raises(ValueError):
        ops.placement_tables(torch.from_numpy(HAND), 0, 2, 3)       # fewer positions than experts


def test_expert_mapping_known_answers_of_the_reference():
    from omni_infer_amd.placement import ExpertMapping, OmniPlanner
    # tests/test_expert_mapping.py:20-25: 2 devices, 2 layers, 4 experts
    pat = np.array([[[1, 0, 1, 0], [0, 1, 0, 1]], [[0, 1, 0, 1], [1, 0, 1, 0]]], dtype=np.int32)
    em = ExpertMapping(pat, device="cpu", rank=0, world_size=2, num_devices_per_host=2, num_experts=4, max_moe_layer_num=2)
    assert em.is_expert_on_current_rank(0, 0, 0, 2) == (True, 0)          # :70-74
    assert em.is_expert_on_current_rank(0, 1, 0, 2) == (False, 1)         # :76-80
    assert em.get_num_of_redundant_experts(0, 2, 0) == 0                  # :92-95
    assert em.get_num_of_redundant_experts(1, 1, 0) == 1                  # :97-100
    assert em.get_total_num_layers() == 2                                 # :108-109
    assert [em.get_local_expert_indices_offset(l, r, 4) for l in (0, 1) for r in (0, 1)] == [0, 2, 0, 2]   # :127-134
    assert em.selector.shape == (2, 4, 1) and em.selector.dtype == torch.int32
    # default deployment past the MoE layers of the pattern (:82-88)
    assert em.is_expert_on_current_rank(5, 1, 0, 2) == (True, 1)
    # tests/test_omni_planner.py:84-99 on the 4-device base pattern (64 experts per device)
    pl = OmniPlanner(device="cpu", rank=0, world_size=4, num_experts=256, max_moe_layer_num=58)
    assert pl.is_expert_on_current_rank(0, 0, 0, 3) == (True, 0)
    assert pl.is_expert_on_current_rank(0, 100, 0, 3) == (False, 64)
    assert pl.is_expert_on_current_rank(0, 1, 1, 2) == (False, 0)
    assert pl.is_expert_on_current_rank(1, 3, 0, 2) == (True, 3)
    assert pl.get_num_of_redundant_experts(0, 63, 0) == 1                 # :101-103
    assert pl.get_max_num_deployed_expert_per_rank() == 64
    assert pl.npu_activation_count.shape == (58, 64) and pl.npu_activation_count.dtype == torch.int64
    assert OmniPlanner.get_deepseek_v3_moe_layer_idx("model.layers.5.mlp.experts") == 2     # :69-71
    assert OmniPlanner.get_deepseek_v3_moe_layer_idx("model.layers.10.mlp.experts") == 7
    assert pl.expert_mapping_on_current_layer(58) is None and pl.is_moe_layer(57)
    with pytest.raises(FileNotFoundError):
        ExpertMapping("nonexistent.npy", device="cpu")                    # test_expert_mapping.py:63-66
    with pytest.raises(ValueError):
        ExpertMapping(pat, device="cpu", world_size=4, num_experts=4, max_moe_layer_num=2)


def test_planner_reads_the_reference_config_keys(tmp_path):
    from omni_infer_amd.placement import OmniPlanner
    pat = np.zeros((4, 2, 16), dtype=np.int32)
    for r in range(4):
        pat[r, :, 4 * r:4 * r + 4] = 1
        pat[r, 0, (4 * r + 6) % 16] = 1          # one redundant copy per device and layer
        pat[r, 1, (4 * r + 9) % 16] = 1
    np.save(tmp_path / "pattern.npy", pat)
    (tmp_path / "config.yaml").write_text('pattern_path: "pattern.npy"\nmax_moe_layer_num: 2\nenable_dump: True\n')
    pl = OmniPlanner(config_file=str(tmp_path / "config.yaml"), device="cpu", rank=2, world_size=4, num_devices_per_host=2,
                     num_experts=16)
    nd = pl.get_max_num_deployed_expert_per_rank() * 4
    assert np.array_equal(pl.selector.squeeze(-1).numpy(), P.selector_table(pat, nd, 2, 2))
    assert pl.enable_dump and pl.max_moe_layer_num == 2
    with pytest.raises(ValueError):
        OmniPlanner(device="cpu", world_size=4, num_experts=16)           # max_moe_layer_num is required


# ------------------------------------------------------------------------------------------ device side
@pytest.mark.gpu
def test_remap_ids_kernel():
    from omni_infer_amd import hip_ops as ops
    g = gen(9)
    for n_map, shape in [(256, (64, 8)), (320, (8192, 8)), (32, (1, 1)), (288, (100_003,))]:
        table = torch.randint(0, 400, (n_map, 1), generator=g).to(torch.int32)
        ids = torch.randint(0, n_map, shape, generator=g).to(torch.int32)
        got = ops.remap_ids(ids.cuda(), table.cuda())
        assert got.shape == ids.shape and got.dtype == torch.int32
        assert np.array_equal(got.cpu().numpy(), P.remap_ids(ids.numpy(), table.numpy()))
    # ids outside the table (dropped assignments) are copied; in place; int64 ids as the reference's tests pass them
    ids = torch.tensor([[0, -1, 5, 31], [32, 7, 1000, 2]], dtype=torch.int32)
    table = (torch.arange(32, dtype=torch.int32) + 100)
    d = ids.cuda()
    ops.remap_ids(d, table.cuda(), out=d)
    assert d.cpu().tolist() == [[100, -1, 105, 131], [32, 107, 1000, 102]]
    got = ops.remap_ids(torch.tensor([[3, 4]], dtype=torch.int64).cuda(), table.cuda())
    assert got.cpu().tolist() == [[103, 104]]
    assert ops.remap_ids(torch.empty(0, 8, dtype=torch.int32).cuda(), table.cuda()).shape == (0, 8)


@pytest.mark.gpu
def test_record_activation_kernel():
    from omni_infer_amd import hip_ops as ops
    g = gen(10)
    mod = int(1e16)
    counts = torch.randint(0, mod, (2, 320), generator=g, dtype=torch.int64)
    counts[0, :3] = torch.tensor([mod - 1, mod - 5, 0])
    add = torch.randint(0, 70000, (320,), generator=g).to(torch.int32)
    add[:3] = torch.tensor([1, 70000, 0])
    d = counts.cuda()
    ops.record_activation(d[0], add.cuda(), mod)
    want = P.record_activation(counts[0].numpy(), add.numpy(), mod)
    assert np.array_equal(d[0].cpu().numpy(), want) and want[:3].tolist() == [0, 69995, 0]
    assert torch.equal(d[1].cpu(), counts[1])                  # the other layer's counters are untouched
    with pytest.raises(ValueError):
        ops.record_activation(d[0], add[:5].cuda(), mod)


@pytest.fixture
def placement_env():
    from omni_infer_amd import config, distributed
    yield types.SimpleNamespace(config=config, dist=distributed)
    config.update_model_extra_config(use_omni_placement=False, enable_moe_expert_parallel=True,
                                     moe_dispatch_combine=True, prefill_dispatch_combine=True)
    distributed.set_virtual_ep(1, 0)


def _placed_block(env, rank, H, I, dispatch_combine=False, shared=True):
    """A DeepseekMoE block of 32 logical experts on 8 ranks (4 each) where every rank deploys one more copy:
    5 positions per rank, 40 positions.  All 32 experts are offered to the weight loader; the pattern decides."""
    from omni_infer_amd.layers.deepseek_moe import DeepseekMoE
    from omni_infer_amd.placement import OmniPlanner
    from omni_infer_amd.quantization.compressed_tensors import AscendCompressedTensorsConfig
    E, world = 32, 8
    pat = np.zeros((world, 2, E), dtype=np.int32)
    for r in range(world):
        pat[r, :, 4 * r:4 * r + 4] = 1
        pat[r, 0, (4 * (r + 3) + 1) % E] = 1       # layer 0: one redundant copy from three ranks on
        pat[r, 1, (4 * (r + 5) + 2) % E] = 1
    env.config.update_model_extra_config(enable_moe_expert_parallel=True, moe_dispatch_combine=dispatch_combine,
                                         prefill_dispatch_combine=dispatch_combine, use_omni_placement=True)
    env.dist.set_virtual_ep(world, rank)
    planner = OmniPlanner(device="cuda", rank=rank, world_size=world, num_devices_per_host=4, num_experts=E,
                          pattern=pat, max_moe_layer_num=2, enable_dump=True)
    cfg = types.SimpleNamespace(hidden_size=H, n_routed_experts=E, num_experts_per_tok=8, moe_intermediate_size=I,
                                n_shared_experts=1 if shared else None, n_group=8, topk_group=4, norm_topk_prob=True,
                                scoring_func="sigmoid", topk_method="noaux_tc", routed_scaling_factor=2.5,
                                hidden_act="silu", first_k_dense_replace=3)
    blk = DeepseekMoE(cfg, AscendCompressedTensorsConfig(ignore=["gate"]), prefix="model.layers.3.mlp", device="cuda",
                      planner=planner)
    lay = Layer(E, H, I, seed=31, shared=shared)
    lay.s13 = lay.s13.to(torch.bfloat16).float()
    lay.s2 = lay.s2.to(torch.bfloat16).float()
    g = gen(81)
    gate_w = torch.randn(E, H, generator=g) * 0.02
    bias = torch.randn(E, generator=g) * 0.01
    blk.gate.weight.data.copy_(gate_w)
    blk.gate.e_score_correction_bias.data.copy_(bias)
    ex = blk.experts
    for e in range(E):
        ex.weight_loader(ex.w13_weight, lay.w13_ckpt[e, :I], "w13_weight", "w1", e)
        ex.weight_loader(ex.w13_weight, lay.w13_ckpt[e, I:], "w13_weight", "w3", e)
        ex.weight_loader(ex.w2_weight, lay.w2_ckpt[e], "w2_weight", "w2", e)
        ex.weight_loader(ex.w13_weight_scale, lay.s13[e, :I].unsqueeze(-1), "w13_weight_scale", "w1", e)
        ex.weight_loader(ex.w13_weight_scale, lay.s13[e, I:].unsqueeze(-1), "w13_weight_scale", "w3", e)
        ex.weight_loader(ex.w2_weight_scale, lay.s2[e].unsqueeze(-1), "w2_weight_scale", "w2", e)
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
    return blk, lay, pat, bias, planner


@pytest.mark.gpu
@pytest.mark.parametrize("rank", [0, 6])
def test_block_with_redundant_placement_against_oracle(placement_env, rank):
    """The block's share under a placement with redundant copies.  The expected output does not use the position
    tables: a token's assignment is computed here iff the rank's selector sends that logical expert to one of the
    rank's own positions, and it is computed with that logical expert's weights.  (Inside one device positions
    ascend with the expert id, so the order of the weighted sum is the same in both.)"""
    H, I, T = 1024, 512, 96
    blk, lay, pat, bias, planner = _placed_block(placement_env, rank, H, I)
    assert blk.local_expert_num == 5 and blk._positions_per_rank() == 5
    x = tokens(T, H, 17)
    xd = x.cuda()
    logits = blk.gate(xd.float())[0].cpu()
    w_ref, ids_ref = O.route_noaux_tc(logits, bias, 8, 8, 4, 2.5)
    sel = P.selector_table(pat, 40, rank, 4)[0]
    assert np.array_equal(planner.selector[0].squeeze(-1).cpu().numpy(), sel)
    pos_ref = torch.from_numpy(P.remap_ids(ids_ref.numpy(), sel))
    w, pos = blk._route(xd)
    assert torch.equal(pos.cpu(), pos_ref) and torch.equal(w.cpu(), w_ref)
    lo = rank * 5
    local = (pos_ref >= lo) & (pos_ref < lo + 5)
    deployed = set(np.nonzero(pat[rank, 0])[0].tolist())
    assert set(ids_ref[local].tolist()) <= deployed and len(deployed) == 5
    ids_masked = torch.where(local, ids_ref, torch.full_like(ids_ref, 32))
    xq, xs = O.dynamic_quant(x)
    want = O.fused_experts_w8a8_allgather_ep(xq, xs, lay.w1_t, lay.w2_t, lay.s13, lay.s2, w_ref, ids_masked, (0, 32))
    want = want + O.shared_expert_mlp(x, *lay.shared)
    out, _ = blk(xd, None, None, 3)
    assert torch.equal(out.float().cpu(), want.float())
    blk.fused = False
    out2, _ = blk(xd, None, None, 3)
    assert torch.equal(out2.float().cpu(), want.float())


@pytest.mark.gpu
def test_one_rank_dispatch_counts_activations(placement_env):
    """The dispatch/combine branch records how many tokens each deployed expert of the rank received."""
    from omni_infer_amd import hip_ops as ops
    H, I, T = 1024, 512, 40
    blk, lay, pat, bias, planner = _placed_block(placement_env, 0, H, I, dispatch_combine=True, shared=False)
    placement_env.dist.set_virtual_ep(1, 0)      # the one-rank form of dispatch/combine
    g = gen(23)
    pos = torch.randint(0, 5, (T, 8), generator=g).to(torch.int32)
    w = torch.rand(T, 8, generator=g)
    x = tokens(T, H, 23)
    for step in range(2):
        blk.experts(x.cuda(), w.cuda(), pos.cuda(), None, None)
    want = torch.bincount(pos.flatten().long(), minlength=5) * 2
    assert torch.equal(planner.npu_activation_count[0].cpu(), want)
    assert int(planner.npu_activation_count[1].abs().sum()) == 0
