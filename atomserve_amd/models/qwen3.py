"""Qwen3 dense decoder (`Qwen3ForCausalLM`): configuration -> layer plan, and the
checkpoint's tensor names (reference atomserve/model.py:292-385, atomserve/loader.py:106-138).

Every layer: RMSNorm, grouped-query attention with a per-head RMSNorm of q and k
before the rotary encoding, RMSNorm, SwiGLU feed-forward; pre-norm residuals; a final
RMSNorm and a head that is the embedding table when the configuration ties them.
"""

import math

from atomserve_amd.config.model_config import Qwen3Config
from atomserve_amd.config.registry import Architecture, register_architecture
from atomserve_amd.parts.plan import (
    AttentionSpec,
    BlockSpec,
    GatedMLPSpec,
    ModelPlan,
    NormSpec,
    RotarySpec,
    sequential_run,
)


def build_plan(c: Qwen3Config) -> ModelPlan:
    def norm(size):
        return NormSpec("rmsnorm", size, c.rms_norm_eps)

    layer = BlockSpec(
        arrangement="prenorm",
        mixer=AttentionSpec(
            kind="attention",
            hidden_size=c.hidden_size,
            num_heads=c.num_heads,
            num_kv_heads=c.num_kv_heads,
            head_dim=c.head_dim,
            scale=1.0 / math.sqrt(c.head_dim),
            qk_norm=norm(c.head_dim),
            position=RotarySpec("rope_half", c.head_dim, c.rope_theta),
            window=0,
        ),
        mixer_norm=norm(c.hidden_size),
        ffn=GatedMLPSpec("gated_mlp", c.hidden_size, c.intermediate_size, "silu"),
        ffn_norm=norm(c.hidden_size),
    )
    return ModelPlan(
        vocab_size=c.vocab_size,
        hidden_size=c.hidden_size,
        layers=tuple(layer for _ in range(c.num_layers)),
        run=sequential_run(c.num_layers),
        final_norm=norm(c.hidden_size),
        tied_head=c.tie_word_embeddings,
        max_positions=c.max_position_embeddings,
    )


def checkpoint_map(c: Qwen3Config) -> dict:
    """Plan tensor name -> checkpoint names, stacked along the output rows in this order:
    q, k, v into one projection, gate, up into one (reference atomserve/loader.py:112-121)."""
    names = {"embed.weight": ["model.embed_tokens.weight"], "final_norm.weight": ["model.norm.weight"]}
    if not c.tie_word_embeddings:
        names["head.weight"] = ["lm_head.weight"]
    for i in range(c.num_layers):
        src, dst = f"model.layers.{i}.", f"layers.{i}."
        names[dst + "mixer_norm.weight"] = [src + "input_layernorm.weight"]
        names[dst + "mixer.qkv.weight"] = [src + f"self_attn.{p}_proj.weight" for p in "qkv"]
        names[dst + "mixer.q_norm.weight"] = [src + "self_attn.q_norm.weight"]
        names[dst + "mixer.k_norm.weight"] = [src + "self_attn.k_norm.weight"]
        names[dst + "mixer.o.weight"] = [src + "self_attn.o_proj.weight"]
        names[dst + "ffn_norm.weight"] = [src + "post_attention_layernorm.weight"]
        names[dst + "ffn.gate_up.weight"] = [src + "mlp.gate_proj.weight", src + "mlp.up_proj.weight"]
        names[dst + "ffn.down.weight"] = [src + "mlp.down_proj.weight"]
    return names


def checkpoint_shapes(c: Qwen3Config) -> dict:
    """Checkpoint name -> (shape, role).  The order is the order of random draws: per layer
    input norm, q, k, v, q norm, k norm, o, post-attention norm, gate, up, down; then the
    embedding, the final norm, and the head if it is not tied."""
    h, q, kv, inter = c.hidden_size, c.num_heads * c.head_dim, c.num_kv_heads * c.head_dim, c.intermediate_size
    shapes = {}
    for i in range(c.num_layers):
        p = f"model.layers.{i}."
        shapes[p + "input_layernorm.weight"] = ((h,), "vector")
        shapes[p + "self_attn.q_proj.weight"] = ((q, h), "matrix")
        shapes[p + "self_attn.k_proj.weight"] = ((kv, h), "matrix")
        shapes[p + "self_attn.v_proj.weight"] = ((kv, h), "matrix")
        shapes[p + "self_attn.q_norm.weight"] = ((c.head_dim,), "vector")
        shapes[p + "self_attn.k_norm.weight"] = ((c.head_dim,), "vector")
        shapes[p + "self_attn.o_proj.weight"] = ((h, q), "matrix")
        shapes[p + "post_attention_layernorm.weight"] = ((h,), "vector")
        shapes[p + "mlp.gate_proj.weight"] = ((inter, h), "matrix")
        shapes[p + "mlp.up_proj.weight"] = ((inter, h), "matrix")
        shapes[p + "mlp.down_proj.weight"] = ((h, inter), "matrix")
    shapes["model.embed_tokens.weight"] = ((c.vocab_size, h), "matrix")
    shapes["model.norm.weight"] = ((h,), "vector")
    if not c.tie_word_embeddings:
        shapes["lm_head.weight"] = ((c.vocab_size, h), "matrix")
    return shapes


def ignored(c: Qwen3Config) -> set:
    """A tied checkpoint may still ship a copy of the head; the configuration decides
    (reference atomserve/loader.py:131-134)."""
    return {"lm_head.weight"} if c.tie_word_embeddings else set()


QWEN3 = register_architecture(
    Architecture(
        name=Qwen3Config.architecture,
        parse_config=Qwen3Config.from_dict,
        build_plan=build_plan,
        checkpoint_map=checkpoint_map,
        checkpoint_shapes=checkpoint_shapes,
        ignored=ignored,
    ),
    replace=True,
)
