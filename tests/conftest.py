"""Shared fixtures: the two tiny Qwen3 configurations and seeded random weights."""

import json
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


# Two configurations that differ in every size and option: head counts and group
# (2 and 3), head_dim (16 and 32, so heads*head_dim equals hidden in A only), sizes
# that are no power of two, layers, vocabulary, eps, theta, tied or untied head.
TINY_A = {
    "architectures": ["Qwen3ForCausalLM"],
    "vocab_size": 256,
    "hidden_size": 64,
    "intermediate_size": 128,
    "num_hidden_layers": 2,
    "num_attention_heads": 4,
    "num_key_value_heads": 2,
    "head_dim": 16,
    "rms_norm_eps": 1e-6,
    "rope_theta": 10000.0,
    "tie_word_embeddings": True,
    "max_position_embeddings": 256,
    "hidden_act": "silu",
}
TINY_B = {
    "architectures": ["Qwen3ForCausalLM"],
    "vocab_size": 1000,
    "hidden_size": 96,
    "intermediate_size": 160,
    "num_hidden_layers": 3,
    "num_attention_heads": 6,
    "num_key_value_heads": 2,
    "head_dim": 32,
    "rms_norm_eps": 1e-5,
    "rope_theta": 1000000.0,
    "tie_word_embeddings": False,
    "max_position_embeddings": 512,
    "hidden_act": "silu",
}
TINY = {"A": TINY_A, "B": TINY_B}


def plain_random_weights(raw: dict, seed: int, std: float = 0.02, gain_std: float = 0.1) -> dict:
    """Checkpoint-named random tensors made by the tests themselves (not by the package):
    matrices N(0, std), norm gains 1 + N(0, gain_std), rounded to bfloat16 values so the
    same numbers are exact in both precisions; returned as float32."""
    g = torch.Generator().manual_seed(seed)
    h, inter = raw["hidden_size"], raw["intermediate_size"]
    H, KV = raw["num_attention_heads"], raw["num_key_value_heads"]
    D = raw.get("head_dim", h // H)

    def mat(*shape):
        return (torch.randn(*shape, generator=g) * std).bfloat16().float()

    def gain(n):
        return (1.0 + torch.randn(n, generator=g) * gain_std).bfloat16().float()

    w = {"model.embed_tokens.weight": mat(raw["vocab_size"], h), "model.norm.weight": gain(h)}
    for i in range(raw["num_hidden_layers"]):
        p = f"model.layers.{i}."
        w[p + "input_layernorm.weight"] = gain(h)
        w[p + "self_attn.q_proj.weight"] = mat(H * D, h)
        w[p + "self_attn.k_proj.weight"] = mat(KV * D, h)
        w[p + "self_attn.v_proj.weight"] = mat(KV * D, h)
        w[p + "self_attn.q_norm.weight"] = gain(D)
        w[p + "self_attn.k_norm.weight"] = gain(D)
        w[p + "self_attn.o_proj.weight"] = mat(h, H * D)
        w[p + "post_attention_layernorm.weight"] = gain(h)
        w[p + "mlp.gate_proj.weight"] = mat(inter, h)
        w[p + "mlp.up_proj.weight"] = mat(inter, h)
        w[p + "mlp.down_proj.weight"] = mat(h, inter)
    if not raw.get("tie_word_embeddings", False):
        w["lm_head.weight"] = mat(raw["vocab_size"], h)
    return w


def write_model_dir(path, raw: dict, weights: dict, dtype=torch.bfloat16):
    """A model folder as a user would have it: config.json and model.safetensors."""
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(raw, f)
    save_file({k: v.to(dtype).contiguous() for k, v in weights.items()},
              os.path.join(path, "model.safetensors"))
    return path


@pytest.fixture(scope="session", params=["A", "B"])
def tiny(request):
    """(name, raw config, checkpoint-named float32 weights) for each tiny configuration."""
    raw = TINY[request.param]
    return request.param, raw, plain_random_weights(raw, seed=11 if request.param == "A" else 23)
