"""CPU-side checks: the built library exports the whole C ABI of include/omni_moe_hip.h, argument
validation of the entry points (no GPU work is enqueued), the flag file, the product path's
refusal to run without the library or on CPU tensors, and that no shipped module touches the oracle."""
import ctypes
import json
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from omni_infer_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from omni_infer_amd import _build
        _build.build(verbose=False)
    return _lib.lib()


def _header_functions(names=("omni_moe_hip.h", "omni_moe_diag.h")):
    found = set()
    for name in names:
        text = open(os.path.join(ROOT, "include", name)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        found |= set(re.findall(r"\b(omni_[a-z0-9_]+)\s*\(", text))
    return sorted(found)


def test_operator_header_lists_operators_only():
    """Measurement helpers live in their own header."""
    ops_only = _header_functions(("omni_moe_hip.h",))
    assert not [n for n in ops_only if n.startswith("omni_diag_") or n in ("omni_moe_reload_tuning", "omni_moe_gemm_kernel_name")]
    assert set(_header_functions(("omni_moe_diag.h",))) == {
        "omni_diag_mfma_i8_rate", "omni_diag_mfma_i8_tile_rate", "omni_diag_hbm_read_rate", "omni_moe_reload_tuning",
        "omni_moe_gemm_kernel_name"}


def test_library_exports_every_declared_symbol(lib):
    from omni_infer_amd import _lib
    names = _header_functions()
    assert len(names) >= 14
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == names
    assert lib.omni_moe_abi_version() == _lib.ABI_VERSION == 7


def test_header_constants_match_binding():
    from omni_infer_amd import _lib
    text = open(os.path.join(ROOT, "include", "omni_moe_hip.h")).read()
    for name, val in re.findall(r"#define\s+(OMNI_[A-Z0-9_]+)\s+\(?(-?\d+)\)?", text):
        if hasattr(_lib, name):
            assert getattr(_lib, name) == int(val), name


def test_argument_validation_returns_codes(lib):
    """Rejected arguments come back as negative codes with a message; nothing is launched."""
    assert lib.omni_moe_route(None, None, 4, 256, 8, 4, 8, 1, 1, 0, 0, 1, 2.5, 1e-20, None, None, None) == -1
    assert b"null" in lib.omni_moe_last_error()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    assert lib.omni_moe_route(p, None, 4, 1024, 1, 1, 8, 1, 1, 0, 0, 1, 1.0, 0.0, p, p, None) == -2   # E > 512
    assert lib.omni_moe_route(p, None, 4, 256, 7, 4, 8, 1, 1, 0, 0, 1, 1.0, 0.0, p, p, None) == -2    # 7 !| 256
    assert lib.omni_moe_route(p, None, 4, 256, 8, 9, 8, 1, 1, 0, 0, 1, 1.0, 0.0, p, p, None) == -1    # topk_group
    assert lib.omni_moe_route(p, None, 0, 256, 8, 4, 8, 1, 1, 0, 0, 1, 1.0, 0.0, p, p, None) == 0     # empty batch
    assert lib.omni_dynamic_quant(p, 7, 4, 64, 64, p, p, None) == -1                                    # dtype
    assert lib.omni_dynamic_quant(p, 0, 4, 64, 32, p, p, None) == -1                                    # ld < cols
    assert lib.omni_dynamic_quant(p, 0, 0, 64, 64, p, p, None) == 0
    assert lib.omni_moe_permute(p, 4, 8, 0, 300, 0, p, p, p, p, p, 1 << 20, None) == -2                 # > 256 local
    assert lib.omni_moe_permute(p, 4, 8, 5, 5, 0, p, p, p, p, p, 1 << 20, None) == -1
    assert lib.omni_moe_permute(p, 4096, 8, 0, 32, 0, p, p, p, p, p, 16, None) == -3                    # workspace
    assert lib.omni_moe_pack_weight(p, 0, 1, 100, 16, p, None) == -2                                    # Kdim % 64
    assert lib.omni_moe_gemm1_swiglu_quant(p, p, None, 0, 4, 1, p, p, None, None, 0, p, 1, 7168, 2000, 4, 0, None, p, p,
                                           None, p, 1 << 30, None) == -2                                # I % 64
    assert lib.omni_moe_gemm1_swiglu_quant(p, p, None, 0, 4, 1, p, p, None, None, 0, p, 1, 7168, 2048, 4, 0, None, p, p,
                                           None, p, 16, None) == -3
    assert lib.omni_moe_gemm1_swiglu_quant(p, p, None, 0, 4, 1, p, p, None, None, 0, p, 1, 7168, 2048, 4, 1, p, p, p,
                                           None, p, 1 << 30, None) == -1            # quant_scale with the bf16 epilogue
    assert lib.omni_moe_group_offsets(p, 0, 300, p, None) == -2                                         # > 256 groups
    assert lib.omni_moe_group_offsets(None, 0, 4, p, None) == -1
    assert lib.omni_moe_gemm2_dequant(p, p, p, p, None, None, 0, p, 1, 7168, 2048, 4, 5, p, None, None, 0, None) == -1
    assert lib.omni_moe_combine(p, 1, p, p, 0, 0, 4, 100, 64, None, None, None, p, None) == -2          # K > 64
    assert lib.omni_moe_w8a8_layer(p, -1, None, p, p, 4, 8, 0, 32, p, p, p, p, None, None, None, None, None, 7168, 2048, 1,
                                   p, p, 1 << 30, None) == -1                                           # int8 w/o scale
    assert lib.omni_moe_w8a8_layer(p, 0, None, p, p, 4, 8, 0, 32, p, p, p, p, None, None, None, None, None, 7168, 2048, 2,
                                   p, p, 1 << 30, None) == -1                                           # rows_dtype f16
    # the whole block: the gate's and the router's checks come first
    block = lambda x_dtype, xq, xs, H, E: lib.omni_moe_w8a8_block(
        p, x_dtype, xq, xs, p, 1, None, E, 8, 4, 1, 1, 0, 0, 1, 2.5, 1e-20, 0, p, p, 4, 8, 0, 32, p, p, p, p, None, None,
        None, None, H, 2048, 1, p, p, 1 << 30, None)
    assert block(1, None, None, 7168, 256) == -2 and b"bf16" in lib.omni_moe_last_error()             # fp32 tokens, not quantised
    assert block(0, p, None, 7168, 256) == -1                                                           # int8 without scales
    assert block(0, None, None, 7168, 1024) == -2                                                       # E > 512
    assert block(0, None, None, 7200, 256) == -2 and b"128" in lib.omni_moe_last_error()              # H % 128
    assert lib.omni_moe_w8a8_block_workspace_bytes(4, 8, 32, 7200, 2048, 256, 1, 1) == 0
    assert lib.omni_moe_w8a8_layer_workspace_bytes(4, 8, 32, 7168, 2048, 1, 2) == 0
    # router and layer in one call: the router's checks come first, then the layer's
    routed = lambda logits, E, n_group, T, rows_dtype: lib.omni_moe_w8a8_layer_routed(
        p, 0, None, logits, None, E, n_group, 4, 1, 1, 0, 0, 1, 2.5, 1e-20, p, p, T, 8, 0, 32, p, p, p, p, None, None,
        None, None, 7168, 2048, rows_dtype, p, p, 1 << 30, None)
    assert routed(None, 256, 8, 4, 1) == -1 and b"null" in lib.omni_moe_last_error()
    assert routed(p, 1024, 8, 4, 1) == -2                                                                # E > 512
    assert routed(p, 256, 7, 4, 1) == -2 and b"n_group" in lib.omni_moe_last_error()
    assert routed(p, 256, 8, 4, 2) == -1                                                                 # rows_dtype f16
    assert routed(p, 256, 8, 0, 1) == 0                                                                  # empty batch
    assert lib.omni_moe_remap_ids(p, -1, p, 32, p, None) == -1
    assert lib.omni_moe_remap_ids(p, 8, None, 32, p, None) == -1
    assert lib.omni_moe_remap_ids(None, 0, None, 32, None, None) == 0                                    # nothing to do
    assert lib.omni_moe_record_activation(p, p, 4, 0, None) == -1                                        # modulus
    assert lib.omni_moe_record_activation(None, p, 4, 10, None) == -1
    assert lib.omni_moe_record_activation(None, None, 0, 10, None) == 0
    assert lib.omni_placement_tables(None, 1, 1, 1, 0, 1, 1, None, p) == -1
    assert lib.omni_diag_hbm_read_rate(None, 1 << 20, 256, p, None) == -1


def test_workspace_sizes(lib):
    assert lib.omni_moe_permute_workspace_bytes(64, 8, 32) == 256
    assert lib.omni_moe_permute_workspace_bytes(8192, 8, 32) == (64 + 1) * 257 * 4
    m_cap = 64 * 8 + 64
    assert lib.omni_moe_gemm1_workspace_bytes(64, 8, 32, 64, m_cap, 7168, 2048) >= m_cap * 2048 * 4 + m_cap * 4
    # prefill-sized: the fp32 y = silu(gate) * up matrix (not the int32 gate/up planes) plus the 64 MiB
    # scratch of the tiles whose reduction is shared between blocks
    big = lib.omni_moe_gemm1_workspace_bytes(8192, 8, 32, 8192, 73728, 7168, 2048)
    assert 73728 * 2048 * 4 + (64 << 20) <= big < 73728 * 2048 * 4 + (65 << 20)
    assert lib.omni_moe_gemm2_workspace_bytes(32, 8192, 73728, 7168, 2048) == (64 << 20) + 8192   # partial sums + the arrival counters of both GEMMs
    assert lib.omni_moe_gemm2_workspace_bytes(32, 64, 576, 7168, 2048) == 0
    from omni_infer_amd import _lib
    total = lib.omni_moe_w8a8_layer_workspace_bytes(64, 8, 32, 7168, 2048, 1, _lib.OMNI_DT_F32)
    assert total >= m_cap * (2048 + 2048 * 4 + 7168 * 4)
    assert total % 256 == 0
    # the row buffer is the caller's choice and nothing else: bf16 rows save exactly half of it, at any size
    for T in (64, 8192):
        f32 = lib.omni_moe_w8a8_layer_workspace_bytes(T, 8, 32, 7168, 2048, 1, _lib.OMNI_DT_F32)
        b16 = lib.omni_moe_w8a8_layer_workspace_bytes(T, 8, 32, 7168, 2048, 1, _lib.OMNI_DT_BF16)
        assert f32 - b16 == (T * 9) * 7168 * 2


def test_python_errors_match_reference_types(lib):
    """ValueError for invalid arguments, RuntimeError for what cannot run (layer.py:224,325,327)."""
    from omni_infer_amd import _lib, hip_ops
    with pytest.raises(ValueError):
        _lib.check(-1, "x")
    with pytest.raises(RuntimeError):
        _lib.check(-2, "x")
    with pytest.raises(RuntimeError, match="GPU only"):
        hip_ops.npu_dynamic_quant(torch.zeros(2, 64, dtype=torch.bfloat16))
    from omni_infer_amd.layers.layer import FusedMoE
    with pytest.raises(ValueError, match="topk_group"):
        FusedMoE.select_experts(None, torch.zeros(2, 8), 2, True, True, None, 4)
    with pytest.raises(ValueError, match="num_expert_group"):
        FusedMoE.select_experts(None, torch.zeros(2, 8), 2, True, True, 2, None)
    from omni_infer_amd.quantization.compressed_tensors import AscendCompressedTensorsConfig
    with pytest.raises(RuntimeError, match="must not be None"):
        FusedMoE(8, 2, 1024, 512, use_grouped_topk=True, quant_config=AscendCompressedTensorsConfig())
    with pytest.raises(ValueError, match="Only softmax"):
        FusedMoE(8, 2, 1024, 512, scoring_func="sigmoid", quant_config=AscendCompressedTensorsConfig(), device="meta")
    with pytest.raises(NotImplementedError):
        AscendCompressedTensorsConfig(num_bits=4)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from omni_infer_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.OmniMoeError, match="no fallback"):
        _lib.lib()


def test_flag_file_roundtrip(tmp_path):
    from omni_infer_amd import config
    f = tmp_path / "cfg.json"
    f.write_text(json.dumps({"model_parallel_config": {"dp_size": 4, "unknown_key": 1},
                             "operator_optimizition_config": {"moe_dispatch_combine": False, "gmm_nz": True,
                                                              "use_mlaprolog": True}}))
    c = config.init_model_extra_config(str(f))
    assert c.parall_config.dp_size == 4 and c.operator_opt_config.moe_dispatch_combine is False
    assert c.operator_opt_config.gmm_nz is True
    assert config.init_model_extra_config(str(tmp_path / "absent.json")).operator_opt_config.moe_dispatch_combine
    bad = tmp_path / "bad.json"
    bad.write_text("{")
    with pytest.raises(RuntimeError, match="Invalid JSON"):
        config.init_model_extra_config(str(bad))
    bad.write_text("{}")
    with pytest.raises(RuntimeError, match="Missing required key"):
        config.init_model_extra_config(str(bad))


def test_weight_loader_places_shards():
    from omni_infer_amd import config, distributed
    from omni_infer_amd.layers.layer import FusedMoE
    from omni_infer_amd.quantization.compressed_tensors import AscendCompressedTensorsConfig
    config.update_model_extra_config(enable_moe_expert_parallel=True)
    distributed.set_virtual_ep(4, 2)
    try:
        m = FusedMoE(16, 2, 128, 64, params_dtype=torch.bfloat16, quant_config=AscendCompressedTensorsConfig())
        assert m.w13_weight.shape == (4, 128, 128) and m.w2_weight.shape == (4, 128, 64)
        assert m.w13_weight_scale.dtype == torch.bfloat16 and m.w13_weight_scale.shape == (4, 128)
        m.w13_weight.data.zero_()
        w1 = torch.full((64, 128), 3, dtype=torch.int8)
        w3 = torch.full((64, 128), 5, dtype=torch.int8)
        m.weight_loader(m.w13_weight, w1, "w13_weight", "w1", 9)      # global 9 = local 1 on rank 2
        m.weight_loader(m.w13_weight, w3, "w13_weight", "w3", 9)
        m.weight_loader(m.w13_weight, w3, "w13_weight", "w3", 3)      # another rank's expert: ignored
        assert bool((m.w13_weight[1, :64] == 3).all()) and bool((m.w13_weight[1, 64:] == 5).all())
        assert bool((m.w13_weight[0] == 0).all()) and bool((m.w13_weight[3] == 0).all())
        m.weight_loader(m.w2_weight_scale, torch.full((128, 1), 0.5), "w2_weight_scale", "w2", 8)
        assert bool((m.w2_weight_scale[0] == 0.5).all())
        with pytest.raises(ValueError, match="shard_id"):
            m.weight_loader(m.w2_weight, w1, "w2_weight", "w9", 8)
    finally:
        distributed.set_virtual_ep(1, 0)


def test_forced_expert_balance(monkeypatch):
    """apply_expert_load_balance with the best_ep flag (reference layer.py:288-297): a prefill instance deals the
    256 expert ids round robin, eight per token, whatever the router chose; a decode instance takes the caller's
    ids when it is given some; without the flag the routing passes through."""
    from omni_infer_amd import config
    from omni_infer_amd.layers.layer import FusedMoE
    from omni_infer_amd.quantization.compressed_tensors import AscendCompressedTensorsConfig
    ids = torch.randint(0, 256, (70, 8), dtype=torch.int32)
    best = torch.randint(0, 256, (70, 8), dtype=torch.int32)
    try:
        m = FusedMoE(8, 2, 128, 64, params_dtype=torch.bfloat16, quant_config=AscendCompressedTensorsConfig())
        assert torch.equal(m.apply_expert_load_balance(ids, best), ids)
        config.update_model_extra_config(best_ep=True)
        assert torch.equal(m.apply_expert_load_balance(ids, best), best)      # decode instance
        assert torch.equal(m.apply_expert_load_balance(ids), ids)
        monkeypatch.setenv("ROLE", "prefill")
        p = FusedMoE(8, 2, 128, 64, params_dtype=torch.bfloat16, quant_config=AscendCompressedTensorsConfig())
        got = p.apply_expert_load_balance(ids, best)
        assert got.shape == ids.shape and got.dtype == torch.int32
        assert torch.equal(got.reshape(-1), torch.arange(70 * 8, dtype=torch.int32) % 256)
        assert int(torch.bincount(got.reshape(-1).long(), minlength=256).max()) <= 70 * 8 // 256 + 1
    finally:
        config.update_model_extra_config(best_ep=False)


def test_product_never_touches_the_oracle():
    """The shipped package must not import, call or read anything under oracle/."""
    pkg = os.path.join(ROOT, "omni_infer_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cc", ".cpp")):
                text = open(os.path.join(base, f)).read()
                assert "oracle" not in text.lower(), f"{f} mentions the oracle"
