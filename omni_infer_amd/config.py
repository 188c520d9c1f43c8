"""Flag file of the MoE path: the mirror of omni/models/common/config/model_config.py.

Only the switches that select a branch of the W8A8 MoE path are kept; their names, defaults
and the JSON layout (``model_parallel_config`` / ``operator_optimizition_config`` read from
``MODEL_EXTRA_CFG_PATH``, model_config.py:81-107, envs.py:55-56) are the reference's.
Unknown keys of a reference flag file are accepted and ignored so that its files load as is.
"""
from __future__ import annotations

import dataclasses
import json
import os
from dataclasses import dataclass, field


@dataclass
class ModelParallelConfig:
    dense_mlp_tp_size: int = 1
    dp_size: int = 1
    o_proj_tp_size: int = 1
    redundancy_shared_expert_num: int = 0


@dataclass
class ModelOperatorOptConfig:
    enable_kv_rmsnorm_rope_cache: bool = True
    prefill_dispatch_combine: bool = True
    moe_multi_stream_tune: bool = False
    best_ep: bool = False
    enable_pd_separated: bool = False
    use_w8a8_dynamic_quant: bool = True
    gmm_nz: bool = False
    moe_dispatch_combine: bool = True
    use_omni_placement: bool = False
    omni_placement_config_path: str = None
    enable_moe_expert_parallel: bool = True
    opt_w2_scale_cast: bool = False
    pd_seperate_prefill: bool = False
    prefill_enable_long_seq: bool = False


@dataclass
class ModelExtraConfig:
    parall_config: ModelParallelConfig = field(default_factory=ModelParallelConfig)
    operator_opt_config: ModelOperatorOptConfig = field(default_factory=ModelOperatorOptConfig)
    model_extra_cfg_path: str = ""


def _known(cls, data: dict) -> dict:
    names = {f.name for f in dataclasses.fields(cls)}
    return {k: v for k, v in data.items() if k in names}


def init_model_extra_config(path: str | None = None) -> ModelExtraConfig:
    path = path if path is not None else os.environ.get("MODEL_EXTRA_CFG_PATH", "")
    cfg = ModelExtraConfig()
    if not path:
        return cfg
    try:
        with open(path, "r") as f:
            data = json.load(f)
        cfg = ModelExtraConfig(
            parall_config=ModelParallelConfig(**_known(ModelParallelConfig, data["model_parallel_config"])),
            operator_opt_config=ModelOperatorOptConfig(
                **_known(ModelOperatorOptConfig, data["operator_optimizition_config"])),
            model_extra_cfg_path=path)
    except FileNotFoundError:
        pass  # the reference warns and keeps the defaults (model_config.py:95-96)
    except json.JSONDecodeError as e:
        raise RuntimeError(f"[ERROR] Invalid JSON format in config file: {e}")
    except KeyError as e:
        raise RuntimeError(f"[ERROR] Missing required key in config data: {e}")
    except TypeError as e:
        raise RuntimeError(f"[ERROR] Config structure mismatch or incorrect field types: {e}")
    return cfg


model_extra_config = init_model_extra_config()


def update_model_extra_config(**kwargs) -> None:
    """Set operator switches by name (model_config.py:116-131)."""
    for key, value in kwargs.items():
        if hasattr(model_extra_config.operator_opt_config, key):
            setattr(model_extra_config.operator_opt_config, key, value)
        elif hasattr(model_extra_config.parall_config, key):
            setattr(model_extra_config.parall_config, key, value)
        else:
            raise KeyError(key)
