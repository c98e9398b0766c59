"""Configuration and registry (CPU)."""

import json

import pytest

from torchllms_amd.config import (
    ARCHITECTURES,
    ConfigError,
    LlamaConfig,
    get_architecture,
    llama_model_spec,
    load_config,
)
from torchllms_amd.config.spec import LayerRun, ModelSpec

from .helpers import TINY_A, TINY_B, TINY_C


def test_reads_config_json_keys():
    cfg = LlamaConfig.from_dict(TINY_B)
    assert (cfg.hidden_size, cfg.num_hidden_layers, cfg.num_attention_heads, cfg.num_key_value_heads) == (256, 3, 8, 1)
    assert cfg.head_dim == 32 and cfg.intermediate_size == 688 and cfg.vocab_size == 512
    assert cfg.rms_norm_eps == 1e-6 and cfg.rope_theta == 500000.0
    assert cfg.rope_scaling.rope_type == "llama3" and cfg.rope_scaling.factor == 8.0
    assert cfg.rope_scaling.original_max_position_embeddings == 64
    assert not cfg.tie_word_embeddings


def test_defaults_follow_the_reference():
    # reference: networks.py:150-154 (head_dim, n_kv_heads), :120 eps, :123 theta
    d = {k: v for k, v in TINY_A.items() if k not in ("num_key_value_heads", "rms_norm_eps", "rope_theta")}
    cfg = LlamaConfig.from_dict(d)
    assert cfg.num_key_value_heads == cfg.num_attention_heads == 4
    assert cfg.head_dim == 16
    assert cfg.rms_norm_eps == 1e-5 and cfg.rope_theta == 10000.0
    assert cfg.rope_scaling.rope_type == "default"


def test_head_dim_apart_from_hidden():
    cfg = LlamaConfig.from_dict(TINY_C)
    assert cfg.head_dim == 48 and cfg.num_attention_heads * cfg.head_dim != cfg.hidden_size
    assert cfg.attention_bias


@pytest.mark.parametrize(
    "patch, match",
    [
        ({"num_key_value_heads": 3}, "not a multiple"),
        ({"head_dim": 15}, "even"),
        ({"hidden_size": 0}, "positive"),
        ({"rope_scaling": {"rope_type": "yarn", "factor": 2.0}}, "not supported"),
        ({"rope_scaling": {"rope_type": "llama3", "factor": 2.0}}, "lacks"),
        ({"hidden_act": "gelu"}, "silu"),
        ({"mlp_bias": True}, "mlp_bias"),
        ({"rms_norm_eps": -1.0}, "positive"),
    ],
)
def test_bad_configs_are_refused(patch, match):
    d = dict(TINY_A)
    d.update(patch)
    with pytest.raises(ConfigError, match=match):
        LlamaConfig.from_dict(d)


def test_missing_keys_are_named():
    d = dict(TINY_A)
    del d["intermediate_size"], d["vocab_size"]
    with pytest.raises(ConfigError, match="intermediate_size.*vocab_size"):
        LlamaConfig.from_dict(d)


def test_rope_parameters_spelling():
    d = dict(TINY_A)
    del d["rope_theta"], d["rope_scaling"]
    d["rope_parameters"] = {"rope_theta": 777.0, "rope_type": "default"}
    assert LlamaConfig.from_dict(d).rope_theta == 777.0


def test_registry_by_name(tmp_path):
    assert "LlamaForCausalLM" in ARCHITECTURES
    with pytest.raises(ConfigError, match="not registered.*LlamaForCausalLM"):
        get_architecture("NoSuchModel")
    (tmp_path / "config.json").write_text(json.dumps(TINY_B))
    arch, cfg = load_config(tmp_path)
    assert arch.name == "LlamaForCausalLM" and cfg.num_hidden_layers == 3
    (tmp_path / "config.json").write_text(json.dumps({k: v for k, v in TINY_B.items() if k != "architectures"}))
    with pytest.raises(ConfigError, match="architectures"):
        load_config(tmp_path)


def test_round_trip(tmp_path):
    cfg = LlamaConfig.from_dict(TINY_C)
    cfg.save(tmp_path)
    _, again = load_config(tmp_path)
    assert again == cfg


def test_model_spec_is_data():
    cfg = LlamaConfig.from_dict(TINY_B)
    spec = llama_model_spec(cfg)
    assert len(spec.layers) == 3 and [r.layer for r in spec.order] == [0, 1, 2]
    m = spec.layers[0].parts["mixer"]
    assert m.kind == "attention" and m.params["num_kv_heads"] == 1 and m.params["head_dim"] == 32
    assert m.params["softmax_scale"] == 32 ** -0.5
    assert m.params["position"].params["scaling"]["factor"] == 8.0
    assert spec.layers[0].parts["ffn"].params["intermediate_size"] == 688
    assert spec.final_norm.params["eps"] == 1e-6
    assert spec.head.params["tied"] is False


def test_order_is_checked():
    cfg = LlamaConfig.from_dict(TINY_A)
    spec = llama_model_spec(cfg)
    bad = ModelSpec(**{**spec.__dict__, "order": [LayerRun(0), LayerRun(5)]})
    with pytest.raises(ValueError, match="names layer 5"):
        bad.validate()
    bad = ModelSpec(**{**spec.__dict__, "order": [LayerRun(0, cache_from=0)]})
    with pytest.raises(ValueError, match="earlier run"):
        bad.validate()
    ok = ModelSpec(**{**spec.__dict__, "order": [LayerRun(0), LayerRun(1), LayerRun(0), LayerRun(1, cache_from=1)]})
    ok.validate()


def test_sizes_no_kernel_takes_are_refused_when_the_model_is_checked():
    """A head size above 256 (no attention kernel takes it) and a width beyond what the norm kernel
    holds in LDS are refused by the parts themselves, with the limit in the message, before any
    tensor exists; the engine asks when it is built (tests/test_gpu_engine.py)."""
    import torch

    from torchllms_amd.parts import Model

    ok = LlamaConfig.from_dict(dict(TINY_B, head_dim=256))
    for dtype in (torch.float32, torch.bfloat16):
        Model(llama_model_spec(ok)).check_sizes(dtype)
    big_head = LlamaConfig.from_dict(dict(TINY_B, head_dim=272))
    with pytest.raises(ValueError, match="head size 272.*up to 256"):
        Model(llama_model_spec(big_head)).check_sizes(torch.bfloat16)
    wide = LlamaConfig.from_dict(dict(TINY_A, hidden_size=40960, num_attention_heads=4, head_dim=16, num_hidden_layers=1))
    with pytest.raises(ValueError, match="rmsnorm: rows of 40960 elements.*1 to 40704"):
        Model(llama_model_spec(wide)).check_sizes(torch.float32)
