"""Configuration from config.json keys and the registries."""

import json

import pytest

from helpers import TINY_A, TINY_B, TINY_C
from tokensprint_amd.config import (ConfigError, Qwen3Config, all_registered_models,
                                    architecture_names, get_architecture, get_model_family,
                                    get_model_repo_id, get_models_from_family,
                                    load_named_config, model_is_registered, resolve_model_name)


def test_every_size_comes_from_the_file():
    a, b = Qwen3Config.from_dict(TINY_A), Qwen3Config.from_dict(TINY_B)
    assert (a.hidden_size, a.num_layers, a.num_heads, a.num_kv_heads, a.head_dim,
            a.intermediate_size, a.vocab_size) == (64, 2, 4, 2, 16, 128, 256)
    assert (b.hidden_size, b.num_layers, b.num_heads, b.num_kv_heads, b.head_dim,
            b.intermediate_size, b.vocab_size) == (96, 3, 8, 2, 32, 160, 389)
    assert (a.rms_norm_eps, a.rope_theta, a.max_position, a.tie_word_embeddings) == \
        (1e-6, 10000.0, 128, True)
    assert (b.rms_norm_eps, b.rope_theta, b.max_position, b.tie_word_embeddings) == \
        (1e-5, 1e6, 256, False)
    assert b.q_width == 256 != b.hidden_size and b.group_size == 4


def test_derived_defaults():
    raw = dict(TINY_A)
    del raw["head_dim"], raw["num_key_value_heads"], raw["tie_word_embeddings"]
    cfg = Qwen3Config.from_dict(raw)
    assert cfg.head_dim == 64 // 4 and cfg.num_kv_heads == 4 and not cfg.tie_word_embeddings


@pytest.mark.parametrize("key", ["hidden_size", "num_hidden_layers", "num_attention_heads",
                                 "intermediate_size", "vocab_size", "rms_norm_eps",
                                 "rope_theta", "max_position_embeddings"])
def test_missing_key_is_named(key):
    raw = dict(TINY_A)
    del raw[key]
    with pytest.raises(ConfigError, match=key):
        Qwen3Config.from_dict(raw)


@pytest.mark.parametrize("patch,match", [
    ({"attention_bias": True}, "attention_bias"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"type": "yarn", "factor": 4}}, "rope_scaling"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"head_dim": 15}, "even"),
    ({"hidden_size": -4}, "positive"),
    ({"layer_types": ["full_attention"]}, "layer_types"),
    ({"layer_types": ["full_attention", "sliding_attention"]}, "sliding_window"),
])
def test_values_the_engine_does_not_run_are_refused(patch, match):
    with pytest.raises(ConfigError, match=match):
        Qwen3Config.from_dict({**TINY_A, **patch})


def test_windows_per_layer():
    c = Qwen3Config.from_dict(TINY_C)
    assert c.layer_windows == (None, 24, 24, None)
    raw = {**TINY_A, "use_sliding_window": True, "sliding_window": 8, "max_window_layers": 1}
    assert Qwen3Config.from_dict(raw).layer_windows == (None, 8)
    # use_sliding_window false: the window size is inert, as in Qwen3's shipped files
    raw = {**TINY_A, "use_sliding_window": False, "sliding_window": 8, "max_window_layers": 1}
    assert Qwen3Config.from_dict(raw).layer_windows == (None, None)


def test_round_trip_through_config_json():
    for raw in (TINY_A, TINY_B, TINY_C):
        cfg = Qwen3Config.from_dict(raw)
        again = Qwen3Config.from_dict(json.loads(json.dumps(cfg.to_dict())))
        assert again == cfg


def test_architecture_registry():
    assert "Qwen3ForCausalLM" in architecture_names()
    arch = get_architecture("Qwen3ForCausalLM")
    spec = arch.build_spec(arch.parse_config(TINY_B))
    assert len(spec.layers) == 3 and spec.width == 96 and spec.head.kind == "head"
    with pytest.raises(ValueError, match="Unsupported architecture 'LlamaForCausalLM'"):
        get_architecture("LlamaForCausalLM")


# short and `family/short` names resolve alike (the reference's
# tests/test_model_registry.py:11-36)
def test_named_models_resolve_short_and_long():
    assert resolve_model_name("qwen3-0.6b") == "qwen3-0.6b"
    assert resolve_model_name("qwen/qwen3-0.6b") == "qwen3-0.6b"
    assert get_model_repo_id("qwen3-0.6b") == get_model_repo_id("qwen/qwen3-0.6b") == "qwen/qwen3-0.6b"
    assert model_is_registered("qwen3-8b") and model_is_registered("qwen/qwen3-32b")
    assert not model_is_registered("meta-llama/qwen3-0.6b")
    assert get_model_family("qwen3-8b") == "qwen"
    assert set(get_models_from_family("qwen")) | set(get_models_from_family("tiny")) \
        == set(all_registered_models())
    assert get_models_from_family("qwen", newest_first=False)[0] == "qwen3-0.6b"
    with pytest.raises(ValueError, match=r"Unsupported model_name 'nope'. Available models: \[.*qwen/qwen3-0.6b"):
        resolve_model_name("nope")


def test_named_0_6b_matches_the_reference_factory():
    # engine/models/qwen/_archs.py:92-125 of the reference
    c = Qwen3Config.from_dict(load_named_config("qwen/qwen3-0.6b"))
    assert (c.hidden_size, c.num_heads, c.num_kv_heads, c.head_dim, c.intermediate_size,
            c.vocab_size, c.num_layers, c.max_position, c.rope_theta, c.rms_norm_eps,
            c.tie_word_embeddings) == (1024, 16, 8, 128, 3072, 151_936, 28, 40960,
                                       1_000_000.0, 1e-6, True)


def test_a_model_registered_by_name_at_run_time(tmp_path):
    # what a user (or a test) adds with register_named_model is found by short and long
    # name like the shipped presets; a short name is unique over all families
    import json
    from helpers import TINY_B
    from tokensprint_amd.config.registry import _NAMED, register_named_model
    preset = tmp_path / "tiny-b.json"
    preset.write_text(json.dumps(TINY_B))
    register_named_model("tiny", "tiny-b", preset)
    try:
        assert resolve_model_name("tiny/tiny-b") == "tiny-b"
        assert not model_is_registered("qwen/tiny-b")
        assert Qwen3Config.from_dict(load_named_config("tiny-b")) == Qwen3Config.from_dict(TINY_B)
        with pytest.raises(ValueError, match="already registered"):
            register_named_model("qwen", "tiny-b", preset)
    finally:
        _NAMED.pop("tiny-b")
    assert not model_is_registered("tiny-b")      # the shipped presets hold real models only
