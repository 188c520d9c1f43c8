"""Checkpoint loading of one MoE block: a synthetic compressed-tensors W8A8 checkpoint with the
reference's tensor names (deepseek_v3.py:800-892) is written to safetensors shards, read back
through ``omni_infer_amd.loader`` and compared, parameter by parameter, with what was written."""
import types

import pytest
import torch

from tests.helpers import Layer, gen


def _write_checkpoint(tmp_path, prefix, E, H, I, seed, with_noise_tensors=True):
    """All E experts + shared expert + gate under `prefix`, split over two files. Returns the dict."""
    from safetensors.torch import save_file
    lay = Layer(E, H, I, seed=seed, shared=True)
    g = gen(seed + 7)
    t = {}
    t[f"{prefix}.gate.weight"] = torch.randn(E, H, generator=g) * 0.02
    t[f"{prefix}.gate.e_score_correction_bias"] = torch.randn(E, generator=g) * 0.01
    for e in range(E):
        base = f"{prefix}.experts.{e}"
        t[f"{base}.gate_proj.weight"] = lay.w13_ckpt[e, :I].contiguous()
        t[f"{base}.up_proj.weight"] = lay.w13_ckpt[e, I:].contiguous()
        t[f"{base}.down_proj.weight"] = lay.w2_ckpt[e].contiguous()
        t[f"{base}.gate_proj.weight_scale"] = lay.s13[e, :I].unsqueeze(-1).to(torch.bfloat16)
        t[f"{base}.up_proj.weight_scale"] = lay.s13[e, I:].unsqueeze(-1).to(torch.bfloat16)
        t[f"{base}.down_proj.weight_scale"] = lay.s2[e].unsqueeze(-1).to(torch.bfloat16)
        for proj, n in (("gate_proj", I), ("up_proj", I), ("down_proj", H)):
            t[f"{base}.{proj}.weight_offset"] = torch.zeros(n, 1, dtype=torch.bfloat16)
    sh = f"{prefix}.shared_experts"
    t[f"{sh}.gate_proj.weight"] = lay.sh13_ckpt[:I].contiguous()
    t[f"{sh}.up_proj.weight"] = lay.sh13_ckpt[I:].contiguous()
    t[f"{sh}.down_proj.weight"] = lay.sh2_ckpt.contiguous()
    t[f"{sh}.gate_proj.weight_scale"] = lay.sh_s13[:I].unsqueeze(-1).to(torch.bfloat16)
    t[f"{sh}.up_proj.weight_scale"] = lay.sh_s13[I:].unsqueeze(-1).to(torch.bfloat16)
    t[f"{sh}.down_proj.weight_scale"] = lay.sh_s2.unsqueeze(-1).to(torch.bfloat16)
    if with_noise_tensors:  # tensors of other modules and layers must be skipped
        t["model.layers.9.mlp.gate.weight"] = torch.zeros(E, H)
        t["model.layers.3.self_attn.rotary_emb.inv_freq"] = torch.zeros(4)
        t["model.norm.weight"] = torch.ones(H)
    names = sorted(t)
    half = len(names) // 2
    paths = [str(tmp_path / "model-00001-of-00002.safetensors"), str(tmp_path / "model-00002-of-00002.safetensors")]
    save_file({k: t[k] for k in names[:half]}, paths[0])
    save_file({k: t[k] for k in names[half:]}, paths[1])
    return lay, t, paths


def _block(E, H, I, device=None):
    from omni_infer_amd.layers.deepseek_moe import DeepseekMoE
    from omni_infer_amd.quantization.compressed_tensors import AscendCompressedTensorsConfig
    cfg = types.SimpleNamespace(hidden_size=H, n_routed_experts=E, num_experts_per_tok=2, moe_intermediate_size=I,
                                n_shared_experts=1, n_group=4, topk_group=2, norm_topk_prob=True,
                                scoring_func="sigmoid", topk_method="noaux_tc", routed_scaling_factor=2.5,
                                hidden_act="silu", first_k_dense_replace=3)
    return DeepseekMoE(cfg, AscendCompressedTensorsConfig(ignore=["gate"]), prefix="model.layers.3.mlp", device=device)


def test_expert_params_mapping_shape():
    from omni_infer_amd.loader import make_expert_params_mapping
    m = make_expert_params_mapping("gate_proj", "down_proj", "up_proj", 3)
    assert len(m) == 9
    assert m[0] == ("experts.w13_", "experts.0.gate_proj.", 0, "w1")
    assert m[1] == ("experts.w2_", "experts.0.down_proj.", 0, "w2")
    assert m[2] == ("experts.w13_", "experts.0.up_proj.", 0, "w3")
    assert m[-1] == ("experts.w13_", "experts.2.up_proj.", 2, "w3")


def test_load_block_from_safetensors_local_share(tmp_path):
    from omni_infer_amd import config, distributed
    from omni_infer_amd.loader import iter_safetensors, load_moe_block
    E, H, I = 8, 128, 64
    config.update_model_extra_config(enable_moe_expert_parallel=True)
    distributed.set_virtual_ep(4, 1)          # this rank owns experts 2 and 3
    try:
        lay, t, paths = _write_checkpoint(tmp_path, "model.layers.3.mlp", E, H, I, seed=5)
        blk = _block(E, H, I)
        for p in blk.parameters():                       # poison: everything must be overwritten
            p.data.fill_(7 if p.dtype == torch.int8 else 7.0)
        loaded = load_moe_block(blk, iter_safetensors(paths), "model.layers.3.mlp", E)
        ex = blk.experts
        assert ex.w13_weight.shape == (2, 2 * I, H)
        assert torch.equal(ex.w13_weight.data, lay.w13_ckpt[2:4])
        assert torch.equal(ex.w2_weight.data, lay.w2_ckpt[2:4])
        assert torch.equal(ex.w13_weight_scale.data, lay.s13[2:4].to(torch.bfloat16))
        assert torch.equal(ex.w2_weight_scale.data, lay.s2[2:4].to(torch.bfloat16))
        assert bool((ex.w13_weight_offset.data == 0).all()) and bool((ex.w2_weight_offset.data == 0).all())
        se = blk.shared_experts
        assert torch.equal(se.gate_up_proj.weight.data, lay.sh13_ckpt)
        assert torch.equal(se.gate_up_proj.weight_scale.data.view(-1), lay.sh_s13.to(torch.bfloat16))
        assert torch.equal(se.down_proj.weight.data, lay.sh2_ckpt)
        assert torch.equal(se.down_proj.weight_scale.data.view(-1), lay.sh_s2.to(torch.bfloat16))
        assert torch.equal(blk.gate.weight.data, t["model.layers.3.mlp.gate.weight"])
        assert torch.equal(blk.gate.e_score_correction_bias.data, t["model.layers.3.mlp.gate.e_score_correction_bias"])
        assert {"experts.w13_weight", "experts.w2_weight", "experts.w13_weight_scale", "experts.w2_weight_scale",
                "shared_experts.gate_up_proj.weight", "shared_experts.down_proj.weight", "gate.weight",
                "gate.e_score_correction_bias"} <= loaded
        assert not any(n.startswith("model.") for n in loaded)
    finally:
        distributed.set_virtual_ep(1, 0)


def test_load_block_shape_mismatch_raises(tmp_path):
    from omni_infer_amd import config, distributed
    from omni_infer_amd.loader import load_moe_block
    config.update_model_extra_config(enable_moe_expert_parallel=True)
    distributed.set_virtual_ep(1, 0)
    blk = _block(4, 128, 64)
    bad = [("model.layers.3.mlp.shared_experts.down_proj.weight", torch.zeros(128, 32, dtype=torch.int8))]
    with pytest.raises(RuntimeError, match="shape"):
        load_moe_block(blk, bad, "model.layers.3.mlp", 4)
    bad = [("model.layers.3.mlp.shared_experts.gate_proj.weight", torch.zeros(64, 100, dtype=torch.int8))]
    with pytest.raises(RuntimeError, match="shape"):
        load_moe_block(blk, bad, "model.layers.3.mlp", 4)
    short = [("model.layers.3.mlp.shared_experts.gate_proj.weight", torch.zeros(32, 128, dtype=torch.int8))]
    with pytest.raises(RuntimeError):     # the narrow() of linear.py:744 refuses a shard that is too short
        load_moe_block(blk, short, "model.layers.3.mlp", 4)


@pytest.mark.gpu
def test_block_loaded_from_checkpoint_matches_oracle(tmp_path):
    """Files -> loader -> process_weights_after_loading -> forward, against the oracle on the same weights."""
    from oracle import moe_oracle as O
    from omni_infer_amd import config, distributed
    from omni_infer_amd.loader import iter_safetensors, load_moe_block
    from tests.helpers import tokens
    E, H, I, K = 8, 1024, 512, 2
    config.update_model_extra_config(enable_moe_expert_parallel=True, moe_dispatch_combine=False,
                                     prefill_dispatch_combine=False)
    distributed.set_virtual_ep(2, 1)          # experts 4..7 are local
    try:
        lay, t, paths = _write_checkpoint(tmp_path, "model.layers.3.mlp", E, H, I, seed=9)
        blk = _block(E, H, I, device="cuda")
        load_moe_block(blk, iter_safetensors(paths), "model.layers.3.mlp", E)
        blk.process_weights_after_loading()
        x = tokens(48, H, 21)
        xd = x.cuda()
        logits = blk.gate(xd.float())[0]
        bias = t["model.layers.3.mlp.gate.e_score_correction_bias"]
        bf = lambda v: v.to(torch.bfloat16).float()
        w_loc = (lay.w1_t[4:8], bf(lay.s13[4:8]), lay.w2_t[4:8], bf(lay.s2[4:8]))
        shared = (lay.shared[0], bf(lay.sh_s13), lay.shared[2], bf(lay.sh_s2))
        out_ref = O.deepseek_moe_forward(x, logits.cpu(), bias, w_loc, shared, K, 4, 2, 2.5, (4, 8))
        out, _ = blk(xd, None, None, 3)
        assert torch.equal(out.float().cpu(), out_ref.float())
    finally:
        distributed.set_virtual_ep(1, 0)


# ----------------------------------------------------------------------------- the checkpoint's quant description
def _quant_description(num_bits=None, ignore=("lm_head",), weights=None, inputs=None, fmt="int-quantized"):
    """A ``quant_model_description.json`` in the layout ``AscendCompressedTensorsConfig.from_config`` parses
    (compressed_tensors.py:183-222): one config group for every ``Linear``, the weights' ``num_bits`` per module."""
    if num_bits is None:
        num_bits = {"self_attn.kv_a_proj_with_mqa": 8, "self_attn.q_a_proj": 8, "mlp.experts": 8, "mlp.shared_experts": 8,
                    "mlp.gate_up_proj": 8, "mlp.down_proj": 8}
    w = {"dynamic": False, "num_bits": num_bits, "strategy": "channel", "symmetric": True, "type": "int",
         "group_size": None}
    a = {"dynamic": True, "num_bits": 8, "strategy": "token", "symmetric": True, "type": "int", "group_size": None}
    w.update(weights or {})
    a.update(inputs or {})
    return {"config_groups": {"group_0": {"input_activations": a, "output_activations": None, "targets": ["Linear"],
                                          "weights": w}},
            "format": fmt, "ignore": list(ignore), "quant_method": "compressed-tensors", "kv_cache_scheme": None,
            "fa_quant_type": None}


def test_quant_config_from_description(tmp_path):
    import json
    from omni_infer_amd.layers.linear import ReplicatedLinear
    from omni_infer_amd.quantization.compressed_tensors import AscendCompressedTensorsConfig as Cfg
    from omni_infer_amd.quantization.compressed_tensors_moe import AscendCompressedTensorsW8A8Int8MoEMethod
    from omni_infer_amd.quantization.compressed_tensors_w8a8_int8 import AscendCompressedTensorsW8A8Int8LinearMethod
    assert Cfg.get_config_filenames() == ["quant_model_description.json"]
    with pytest.raises(ValueError, match="quant_model_description.json"):
        Cfg.from_checkpoint_dir(str(tmp_path))
    (tmp_path / "quant_model_description.json").write_text(json.dumps(_quant_description(ignore=["lm_head", "re:.*mlp\\.gate$"])))
    cfg = Cfg.from_checkpoint_dir(str(tmp_path))
    assert list(cfg.target_scheme_map) == ["Linear"] and cfg.quant_format == "int-quantized"
    assert isinstance(cfg.target_scheme_map["Linear"]["weights"].num_bits, dict)       # kept as written
    # scheme selection: per-module bits looked up by the layer's name
    method, bits = cfg.get_moe_method("model.layers.3.mlp.experts")
    assert isinstance(method, AscendCompressedTensorsW8A8Int8MoEMethod) and bits == 8
    lin = ReplicatedLinear(128, 64, bias=False, quant_config=None, prefix="x")
    assert isinstance(cfg.get_quant_method(lin, "model.layers.3.mlp.shared_experts.down_proj"),
                      AscendCompressedTensorsW8A8Int8LinearMethod)
    assert cfg.get_quant_method(lin, "model.layers.3.mlp.gate") is None                  # regex entry of ignore
    assert cfg.get_quant_method(lin, "lm_head") is None                                  # exact entry
    assert cfg.get_quant_method(torch.nn.ReLU(), "model.layers.3.act") is None           # neither linear nor MoE
    with pytest.raises(ValueError, match="weight name mismatch"):                        # a module the dict does not name
        cfg.get_quant_method(lin, "model.layers.3.self_attn.o_proj")
    # anything but dynamic per-token W8A8 is refused where the reference refuses it
    for bad in (dict(weights={"symmetric": False}), dict(inputs={"dynamic": False}), dict(inputs={"strategy": "tensor"}),
                dict(weights={"dynamic": True}), dict(fmt="pack-quantized"), dict(num_bits=16)):
        c = Cfg.from_config(_quant_description(**bad))
        with pytest.raises(NotImplementedError):
            c.get_quant_method(lin, "model.layers.3.mlp.shared_experts.down_proj")
    c4 = Cfg.from_config(_quant_description(num_bits={"mlp.experts": 4, "mlp.shared_experts": 8}))
    m4, b4 = c4.get_moe_method("model.layers.3.mlp.experts")
    assert b4 == 4 and type(m4).__name__ == "AscendCompressedTensorsW4A8Int8MoEMethod"  # empty upstream as well
    with pytest.raises(RuntimeError, match="Unsupported FusedMoe scheme"):
        Cfg.from_config(_quant_description(num_bits=16)).get_moe_method("model.layers.3.mlp.experts")
    # targets: a full layer name and a regex come before the class-name match
    d = _quant_description()
    d["config_groups"]["group_1"] = dict(d["config_groups"]["group_0"], targets=["re:.*down_proj$"],
                                         input_activations=dict(d["config_groups"]["group_0"]["input_activations"], dynamic=False))
    c = Cfg.from_config(d)
    with pytest.raises(NotImplementedError):                                             # the regex group is static
        c.get_quant_method(lin, "model.layers.3.mlp.shared_experts.down_proj")
    assert c.get_quant_method(lin, "model.layers.3.mlp.shared_experts.gate_up_proj") is not None
    # the keyword form used in code keeps meaning the built scheme, and refuses others at once
    assert Cfg(ignore=["gate"]).get_moe_method("x")[1] == 8
    with pytest.raises(NotImplementedError):
        Cfg(num_bits=4)
    with pytest.raises(NotImplementedError):
        Cfg(dynamic=False)


@pytest.mark.gpu
def test_block_configured_and_loaded_from_a_checkpoint_directory(tmp_path):
    """A checkpoint directory as it ships: ``quant_model_description.json`` next to the safetensors shards.  The
    description configures the block (the gate is in ``ignore``), the loader fills it, the forward matches the
    oracle bit for bit."""
    import json
    from oracle import moe_oracle as O
    from omni_infer_amd import config, distributed
    from omni_infer_amd.layers.deepseek_moe import DeepseekMoE
    from omni_infer_amd.loader import iter_safetensors, load_moe_block
    from omni_infer_amd.quantization.compressed_tensors import AscendCompressedTensorsConfig
    from tests.helpers import tokens
    E, H, I, K = 8, 1024, 512, 2
    config.update_model_extra_config(enable_moe_expert_parallel=True, moe_dispatch_combine=False,
                                     prefill_dispatch_combine=False)
    distributed.set_virtual_ep(2, 0)          # experts 0..3 are local
    try:
        lay, t, paths = _write_checkpoint(tmp_path, "model.layers.5.mlp", E, H, I, seed=19)
        (tmp_path / "quant_model_description.json").write_text(json.dumps(_quant_description(ignore=["lm_head", "gate"])))
        qc = AscendCompressedTensorsConfig.from_checkpoint_dir(str(tmp_path))
        mc = types.SimpleNamespace(hidden_size=H, n_routed_experts=E, num_experts_per_tok=K, moe_intermediate_size=I,
                                   n_shared_experts=1, n_group=4, topk_group=2, norm_topk_prob=True, scoring_func="sigmoid",
                                   topk_method="noaux_tc", routed_scaling_factor=2.5, hidden_act="silu",
                                   first_k_dense_replace=3)
        blk = DeepseekMoE(mc, qc, prefix="model.layers.5.mlp", device="cuda")
        assert blk.experts.num_bits == 8 and blk.gate.quant_method is None
        load_moe_block(blk, iter_safetensors(paths), "model.layers.5.mlp", E)
        blk.process_weights_after_loading()
        x = tokens(40, H, 23)
        xd = x.cuda()
        logits = blk.gate(xd.float())[0]
        bias = t["model.layers.5.mlp.gate.e_score_correction_bias"]
        bf = lambda v: v.to(torch.bfloat16).float()
        w_loc = (lay.w1_t[0:4], bf(lay.s13[0:4]), lay.w2_t[0:4], bf(lay.s2[0:4]))
        shared = (lay.shared[0], bf(lay.sh_s13), lay.shared[2], bf(lay.sh_s2))
        out_ref = O.deepseek_moe_forward(x, logits.cpu(), bias, w_loc, shared, K, 4, 2, 2.5, (0, 4))
        out, _ = blk(xd, None, None, 5)
        assert torch.equal(out.float().cpu(), out_ref.float())
    finally:
        distributed.set_virtual_ep(1, 0)
