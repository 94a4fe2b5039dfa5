"""Configuration and registry: every number comes from config.json, and what the engine
does not compute is refused (reference atomserve/config.py:31-92, tests/test_model_unit.py:96-99)."""

import dataclasses
import json

import pytest

from atomserve_amd.config import (
    Architecture,
    ConfigError,
    EngineConfig,
    Qwen3Config,
    architecture_for,
    load_model_config,
    register_architecture,
    supported_architectures,
)
from tests.conftest import TINY_A, TINY_B


@pytest.mark.parametrize("raw", [TINY_A, TINY_B])
def test_every_field_is_read_from_config_json(raw):
    c = Qwen3Config.from_dict(raw)
    assert (c.vocab_size, c.hidden_size, c.intermediate_size, c.num_layers) == (
        raw["vocab_size"], raw["hidden_size"], raw["intermediate_size"], raw["num_hidden_layers"])  # fmt: skip
    assert (c.num_heads, c.num_kv_heads, c.head_dim) == (
        raw["num_attention_heads"], raw["num_key_value_heads"], raw["head_dim"])  # fmt: skip
    assert (c.rms_norm_eps, c.rope_theta, c.tie_word_embeddings, c.max_position_embeddings) == (
        raw["rms_norm_eps"], raw["rope_theta"], raw["tie_word_embeddings"], raw["max_position_embeddings"])  # fmt: skip
    assert Qwen3Config.from_dict(c.to_dict()) == c


def test_the_plan_carries_the_configurations_numbers_to_every_part():
    """The two tiny configurations differ in every size and option; so must their plans."""
    plans = []
    for raw in (TINY_A, TINY_B):
        arch = architecture_for(raw)
        c = arch.parse_config(raw)
        plan = arch.build_plan(c)
        layer = plan.layers[0]
        assert len(plan.layers) == len(plan.run) == c.num_layers
        assert (layer.mixer.num_heads, layer.mixer.num_kv_heads, layer.mixer.head_dim) == (c.num_heads, c.num_kv_heads, c.head_dim)
        assert layer.mixer.scale == pytest.approx(c.head_dim**-0.5)
        assert layer.mixer.qk_norm.eps == layer.mixer_norm.eps == layer.ffn_norm.eps == plan.final_norm.eps == c.rms_norm_eps
        assert layer.mixer.position.theta == c.rope_theta and layer.mixer.position.rotary_dim == c.head_dim
        assert layer.ffn.intermediate_size == c.intermediate_size and layer.ffn.hidden_size == c.hidden_size
        assert plan.tied_head == c.tie_word_embeddings and plan.vocab_size == c.vocab_size
        plans.append(plan)
    a, b = plans
    for field in ("num_heads", "head_dim", "scale"):
        assert getattr(a.layers[0].mixer, field) != getattr(b.layers[0].mixer, field)
    assert a.final_norm.eps != b.final_norm.eps and a.tied_head != b.tied_head


def test_head_dim_defaults_to_hidden_over_heads():
    raw = {k: v for k, v in TINY_A.items() if k != "head_dim"}
    assert Qwen3Config.from_dict(raw).head_dim == 64 // 4


def test_other_architectures_are_refused():
    with pytest.raises(ValueError, match="only supports"):
        architecture_for({"architectures": ["LlamaForCausalLM"]})
    with pytest.raises(ConfigError, match="only supports"):
        architecture_for({})
    assert "Qwen3ForCausalLM" in supported_architectures()


@pytest.mark.parametrize("key,value,match", [
    ("attention_bias", True, "attention_bias"),
    ("rope_scaling", {"type": "yarn"}, "rope_scaling"),
    ("use_sliding_window", True, "use_sliding_window"),
    ("hidden_act", "gelu", "hidden_act"),
])  # fmt: skip
def test_options_that_change_the_math_are_refused(key, value, match):
    with pytest.raises(ConfigError, match=match):
        Qwen3Config.from_dict({**TINY_A, key: value})


def test_missing_keys_are_named():
    raw = {k: v for k, v in TINY_A.items() if k not in ("rope_theta", "vocab_size")}
    with pytest.raises(ConfigError, match="vocab_size.*rope_theta|rope_theta.*vocab_size"):
        Qwen3Config.from_dict(raw)


def test_impossible_sizes_are_refused():
    with pytest.raises(ConfigError, match="multiple"):
        Qwen3Config.from_dict({**TINY_A, "num_attention_heads": 5, "num_key_value_heads": 2})
    with pytest.raises(ConfigError, match="even"):
        Qwen3Config.from_dict({**TINY_A, "head_dim": 15})


def test_load_model_config_reads_the_folder(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(TINY_B))
    arch, c = load_model_config(str(tmp_path))
    assert arch.name == "Qwen3ForCausalLM" and c.hidden_size == 96
    with pytest.raises(FileNotFoundError):
        load_model_config(str(tmp_path / "nothing"))


def test_another_architecture_is_one_registration():
    arch = architecture_for(TINY_A)
    toy = dataclasses.replace(arch, name="ToyForCausalLM")
    register_architecture(toy, replace=True)
    assert architecture_for({**TINY_A, "architectures": ["ToyForCausalLM"]}) is toy
    with pytest.raises(ValueError, match="already registered"):
        register_architecture(Architecture("ToyForCausalLM", None, None, None, None))


def test_engine_config_checks():
    # reference atomserve/config.py:82-92
    assert EngineConfig().block_size == 16 and EngineConfig().max_num_batched_tokens == 512
    with pytest.raises(ValueError, match="exceeds KV pool capacity"):
        EngineConfig(num_blocks=4, block_size=16, max_model_len=65)
    with pytest.raises(ValueError, match="max_num_batched_tokens"):
        EngineConfig(max_num_seqs=32, max_num_batched_tokens=16)
