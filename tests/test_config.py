"""Configuration, registry and model plan (no GPU)."""

import json

import pytest

from dryft_amd.config import ConfigError, Qwen3Config, Run, read_config_json
from dryft_amd.models import known_architectures, register_architecture, resolve_architecture
from dryft_amd.models import load_preset, preset_names
from dryft_amd.models.qwen3 import qwen3_plan
from helpers import TINY_A, TINY_B


def test_reads_every_size_from_the_file():
    cfg = Qwen3Config.from_dict(TINY_B)
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads) == (3, 96, 8, 2)
    assert (cfg.head_dim, cfg.intermediate_size, cfg.vocab_size) == (32, 224, 384)
    assert cfg.rope_theta == 1e6 and cfg.rms_norm_eps == 1e-5 and cfg.tie_word_embeddings is False
    assert (cfg.q_dim, cfg.kv_dim, cfg.group) == (256, 64, 4)          # q width differs from hidden


def test_head_sizes_are_checked_with_everything_else():
    """Any even head size up to 256 is a valid configuration (float32 and bfloat16 both run it); an odd or too
    wide one is one more line of the one error."""
    assert Qwen3Config.from_dict(dict(TINY_A, head_dim=40)).head_dim == 40
    assert Qwen3Config.from_dict(dict(TINY_A, head_dim=72)).q_dim == 4 * 72
    with pytest.raises(ConfigError) as e:
        Qwen3Config.from_dict(dict(TINY_A, head_dim=258, hidden_act="gelu"))
    assert len(e.value.problems) == 2 and any("head_dim" in p and "256" in p for p in e.value.problems)
    with pytest.raises(ConfigError, match="even"):
        Qwen3Config.from_dict(dict(TINY_A, head_dim=33))


def test_head_dim_defaults_to_hidden_over_heads():
    raw = dict(TINY_A)
    del raw["head_dim"]
    assert Qwen3Config.from_dict(raw).head_dim == 64 // 4
    raw["head_dim"] = 0
    assert Qwen3Config.from_dict(raw).head_dim == 16
    raw = dict(TINY_A)
    del raw["tie_word_embeddings"]
    assert Qwen3Config.from_dict(raw).tie_word_embeddings is False      # reference default (config.py:153)


def test_optional_keys_and_model_type_fallback():
    raw = {k: v for k, v in TINY_B.items() if k not in ("max_position_embeddings", "hidden_act", "attention_bias",
                                                        "architectures")}
    cfg = Qwen3Config.from_dict(raw)
    assert cfg.max_position_embeddings is None and "max_position_embeddings" not in cfg.to_dict()
    assert resolve_architecture(raw).name == "Qwen3ForCausalLM"          # found through model_type "qwen3"
    del raw["num_key_value_heads"]
    assert Qwen3Config.from_dict(raw).num_key_value_heads == 8            # as many kv heads as query heads


def test_one_error_lists_every_problem():
    raw = dict(TINY_B, hidden_act="gelu", attention_bias=True, rope_scaling={"type": "yarn"}, use_sliding_window=True,
               num_key_value_heads=3, rms_norm_eps="tiny")
    del raw["vocab_size"]
    with pytest.raises(ConfigError) as e:
        Qwen3Config.from_dict(raw)
    text = str(e.value)
    for key in ("hidden_act", "attention_bias", "rope_scaling", "use_sliding_window", "vocab_size: missing",
                "rms_norm_eps", "not a multiple"):
        assert key in text, key
    assert len(e.value.problems) == 7


def test_round_trip_through_config_json(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_B)
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
    raw = read_config_json(str(tmp_path))
    assert Qwen3Config.from_dict(raw) == cfg
    assert resolve_architecture(raw).name == "Qwen3ForCausalLM"
    with pytest.raises(FileNotFoundError):
        read_config_json(str(tmp_path / "nowhere"))


def test_registry_knows_the_architecture_and_refuses_others():
    assert "Qwen3ForCausalLM" in known_architectures()
    arch = resolve_architecture(TINY_A)
    assert arch.config_class is Qwen3Config
    for bad in ({}, {"architectures": []}, {"architectures": ["LlamaForCausalLM"]}, {"architectures": "Qwen3ForCausalLM"}):
        with pytest.raises(ConfigError) as e:
            resolve_architecture(bad)
        assert "Qwen3ForCausalLM" in str(e.value)                      # the error names what is known
    with pytest.raises(ValueError):
        register_architecture("Qwen3ForCausalLM", Qwen3Config, qwen3_plan)


def test_presets_are_config_files():
    assert {"tiny-a", "tiny-b", "qwen3-4b", "qwen3-8b", "qwen3-32b"} <= set(preset_names())
    cfg = Qwen3Config.from_dict(load_preset("qwen3-4b"))
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.q_dim, cfg.kv_dim, cfg.intermediate_size, cfg.vocab_size) == \
        (36, 2560, 4096, 1024, 9728, 151936)
    assert cfg.tie_word_embeddings and cfg.rope_theta == 5e6
    with pytest.raises(KeyError):
        load_preset("qwen3-1t")


def test_plan_is_data_chosen_layer_by_layer():
    cfg = Qwen3Config.from_dict(TINY_B)
    plan = qwen3_plan(cfg)
    plan.validate()
    assert len(plan.layers) == 3 and plan.schedule == tuple(Run(i, i) for i in range(3))
    layer = plan.layers[1]
    assert layer.block == "prenorm" and set(layer.parts) == {"mixer_norm", "mixer", "ffn_norm", "ffn"}
    mixer = layer.parts["mixer"]
    assert mixer.kind == "gqa_attention" and mixer.args["head_dim"] == 32 and mixer.args["qk_norm_eps"] == 1e-5
    assert mixer.tensors["q_norm"] == "model.layers.1.self_attn.q_norm.weight"
    assert plan.head.tensors == {"weight": "lm_head.weight"}
    assert plan.optional_tensors == {} and plan.max_positions == 4096
    tied = qwen3_plan(Qwen3Config.from_dict(TINY_A))                    # tied: the head reads the embedding's tensor
    assert tied.head.tensors == tied.embedding.tensors == {"weight": "model.embed_tokens.weight"}
    assert tied.optional_tensors == {"lm_head.weight": "model.embed_tokens.weight"}


def test_plan_validation_catches_bad_schedules():
    from dataclasses import replace
    plan = qwen3_plan(Qwen3Config.from_dict(TINY_A))
    with pytest.raises(ValueError, match="names layer"):
        replace(plan, schedule=(Run(0, 0), Run(5, 1))).validate()
    with pytest.raises(ValueError, match="both write"):
        replace(plan, schedule=(Run(0, 0), Run(1, 0))).validate()
    with pytest.raises(ValueError, match="before any run has written"):
        replace(plan, schedule=(Run(0, 1, writes_cache=False), Run(1, 1))).validate()
    replace(plan, schedule=(Run(0, 0), Run(1, 1), Run(1, 2), Run(0, 0, writes_cache=False))).validate()
