"""Pins the plain implementation by what fixes it beside the reference's text: library
routines it must reduce to, vectors from the reference's own tests, and invariants,
each chosen so that a plausible mistake fails it."""

import math

import pytest
import torch
import torch.nn.functional as F

from tests import plain_qwen3 as plain
from tests.conftest import TINY_A, TINY_B, plain_random_weights

torch.manual_seed(0)
F64 = torch.float64


def test_rms_norm_is_the_library_routine():
    x, w = torch.randn(5, 24, dtype=F64) * 3, torch.randn(24, dtype=F64) + 1
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), F.rms_norm(x, (24,), w, 1e-5), atol=1e-12)


def test_rms_norm_unit_rms_and_per_channel_weight():
    # reference tests/test_model_unit.py:15-26
    x = torch.randn(4, 64, dtype=F64) * 7.0
    out = plain.rms_norm(x, torch.ones(64, dtype=F64), 1e-6)
    assert torch.allclose(out.pow(2).mean(-1).sqrt(), torch.ones(4, dtype=F64), atol=1e-5)
    w = torch.arange(1.0, 9.0, dtype=F64)
    y = torch.randn(3, 8, dtype=F64)
    assert torch.allclose(plain.rms_norm(y, w, 1e-6), plain.rms_norm(y, torch.ones(8, dtype=F64), 1e-6) * w)


def test_rms_norm_eps_is_inside_the_root():
    # With x = 0 the result is 0 / sqrt(eps); with tiny x the eps term dominates.
    x = torch.full((1, 4), 1e-4, dtype=F64)
    out = plain.rms_norm(x, torch.ones(4, dtype=F64), 1e-2)
    assert torch.allclose(out, x / math.sqrt(1e-8 + 1e-2))


def test_rope_known_vector_pins_sign_and_pairing():
    # A unit vector on coordinate 0 of a 4-wide head: its partner is coordinate 2 (i + D/2),
    # and it turns counter-clockwise: (cos a, 0, sin a, 0) with a = position * theta^0.
    x = torch.zeros(1, 1, 4, dtype=F64)
    x[0, 0, 0] = 1.0
    out = plain.rope(x, torch.tensor([3]), 100.0)
    assert torch.allclose(out[0, 0], torch.tensor([math.cos(3.0), 0.0, math.sin(3.0), 0.0], dtype=F64))
    # Coordinate 1 pairs with 3 and turns by position * theta^(-2/4) = 3 / 10.
    y = torch.zeros(1, 1, 4, dtype=F64)
    y[0, 0, 1] = 1.0
    out = plain.rope(y, torch.tensor([3]), 100.0)
    assert torch.allclose(out[0, 0], torch.tensor([0.0, math.cos(0.3), 0.0, math.sin(0.3)], dtype=F64))


def test_rope_is_complex_multiplication_of_the_pairs():
    x = torch.randn(6, 3, 16, dtype=F64)
    pos = torch.tensor([0, 1, 5, 300, 4097, 39999])
    ang = plain.rope_angles(pos, 16, 1e6)  # [T, 8]
    z = torch.complex(x[..., :8], x[..., 8:]) * torch.polar(torch.ones_like(ang), ang)[:, None, :]
    assert torch.allclose(plain.rope(x, pos, 1e6), torch.cat([z.real, z.imag], dim=-1), atol=1e-12)


def test_rope_identity_length_and_relative_distance():
    # reference tests/test_model_unit.py:29-52
    x = torch.randn(1, 2, 16, dtype=F64)
    assert torch.allclose(plain.rope(x, torch.tensor([0]), 1e4), x)
    y = torch.randn(5, 3, 16, dtype=F64)
    assert torch.allclose(plain.rope(y, torch.arange(100, 105), 1e4).norm(dim=-1), y.norm(dim=-1))
    q, k = torch.randn(1, 1, 16, dtype=F64), torch.randn(1, 1, 16, dtype=F64)

    def score(m, n):
        return float((plain.rope(q, torch.tensor([m]), 1e4) * plain.rope(k, torch.tensor([n]), 1e4)).sum())

    assert score(7, 3) == pytest.approx(score(107, 103), abs=1e-9)
    assert score(7, 3) != pytest.approx(score(3, 7), abs=1e-3)  # the sign of the distance counts


def test_attention_without_mask_is_the_library_routine():
    # One head, one query at the last position: plain softmax attention.
    q, k, v = torch.randn(1, 1, 8, dtype=F64), torch.randn(9, 1, 8, dtype=F64), torch.randn(9, 1, 8, dtype=F64)
    ours = plain.causal_attention(q, k, v, torch.tensor([8]))
    lib = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1))
    assert torch.allclose(ours, lib.transpose(0, 1), atol=1e-12)


def test_attention_causal_with_groups_is_the_library_routine():
    # 6 query heads over 2 kv heads: head h reads kv head h // 3 (repeat_interleave, as in
    # reference tests/test_model_unit.py:55-64); a fresh sequence has the lower-triangular mask.
    q, k, v = torch.randn(7, 6, 8, dtype=F64), torch.randn(7, 2, 8, dtype=F64), torch.randn(7, 2, 8, dtype=F64)
    ours = plain.causal_attention(q, k, v, torch.arange(7))
    kk, vv = k.repeat_interleave(3, dim=1), v.repeat_interleave(3, dim=1)
    lib = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), is_causal=True)
    assert torch.allclose(ours, lib.transpose(0, 1), atol=1e-12)
    # token 0 sees only itself (reference tests/test_model_unit.py:78-82)
    assert torch.allclose(ours[0], v[0].repeat_interleave(3, dim=0))
    # queries at the end over all keys equal the rows of the full result (:85-93)
    assert torch.allclose(plain.causal_attention(q[4:], k, v, torch.arange(4, 7)), ours[4:], atol=1e-12)


def test_attention_window_hides_old_keys():
    q, k, v = torch.randn(6, 1, 4, dtype=F64), torch.randn(6, 1, 4, dtype=F64), torch.randn(6, 1, 4, dtype=F64)
    out = plain.causal_attention(q, k, v, torch.arange(6), window=1)
    assert torch.allclose(out, v)  # a window of one key is the token itself


def test_swiglu_is_the_library_routine():
    x = torch.randn(4, 12, dtype=F64)
    g, u, d = torch.randn(20, 12, dtype=F64), torch.randn(20, 12, dtype=F64), torch.randn(12, 20, dtype=F64)
    assert torch.allclose(plain.swiglu(x, g, u, d), F.linear(F.silu(F.linear(x, g)) * F.linear(x, u), d), atol=1e-12)


@pytest.mark.parametrize("raw", [TINY_A, TINY_B])
def test_model_shapes_head_tying_and_prefix_property(raw):
    w = plain_random_weights(raw, seed=5, std=0.2, gain_std=0.2)
    ids = torch.randint(0, raw["vocab_size"], (13,)).tolist()
    full = plain.logits(raw, w, ids)
    assert full.shape == (13, raw["vocab_size"])
    # Causality: the logits of a prefix do not depend on what follows.
    assert torch.allclose(plain.logits(raw, w, ids[:6]), full[:6], atol=1e-10)
    # The head is the embedding when tied, and lm_head.weight otherwise.
    if raw["tie_word_embeddings"]:
        other = dict(w)
        other["lm_head.weight"] = torch.randn(raw["vocab_size"], raw["hidden_size"])
        assert torch.equal(plain.logits(raw, other, ids), full)
    else:
        other = dict(w)
        other["lm_head.weight"] = w["lm_head.weight"] * 2
        assert torch.allclose(plain.logits(raw, other, ids), full * 2)


def test_shifting_every_position_changes_nothing():
    # Only distances enter the scores, so a sequence placed at positions 500.. gives the
    # same logits (this fails if v were rotated, or if q and k turned in opposite senses).
    w = plain_random_weights(TINY_B, seed=9, std=0.2, gain_std=0.2)
    ids = torch.randint(0, 1000, (11,)).tolist()
    assert torch.allclose(plain.logits(TINY_B, w, ids), plain.logits(TINY_B, w, ids, position_offset=500), atol=1e-9)


def test_qk_norm_sits_before_the_rotation_and_uses_the_layer_eps():
    # One layer, one head; if the q/k norm came after the rotation, non-uniform gains would
    # act on rotated coordinates and the scores below would change.
    raw = dict(TINY_A, num_hidden_layers=1)
    w = plain_random_weights(raw, seed=2, std=0.3, gain_std=0.4)
    x = torch.randn(5, raw["hidden_size"], dtype=F64)
    pos = torch.arange(5)
    H, KV, D = 4, 2, 16
    wd = {k: v.to(F64) for k, v in w.items()}
    out = plain.attention_layer(x, wd, "model.layers.0.", plain.normalise_config(raw), pos)
    q = F.rms_norm((x @ wd["model.layers.0.self_attn.q_proj.weight"].T).view(5, H, D), (D,),
                   wd["model.layers.0.self_attn.q_norm.weight"], raw["rms_norm_eps"])
    k = F.rms_norm((x @ wd["model.layers.0.self_attn.k_proj.weight"].T).view(5, KV, D), (D,),
                   wd["model.layers.0.self_attn.k_norm.weight"], raw["rms_norm_eps"])
    v = (x @ wd["model.layers.0.self_attn.v_proj.weight"].T).view(5, KV, D)
    q, k = plain.rope(q, pos, raw["rope_theta"]), plain.rope(k, pos, raw["rope_theta"])
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), k.repeat_interleave(2, 1).transpose(0, 1),
                                         v.repeat_interleave(2, 1).transpose(0, 1), is_causal=True)
    ref = ref.transpose(0, 1).reshape(5, H * D) @ wd["model.layers.0.self_attn.o_proj.weight"].T
    assert torch.allclose(out, ref, atol=1e-10)


def test_sampling_distribution_rules():
    # reference tests/test_sampler.py:28-47
    probs = torch.tensor([0.4, 0.3, 0.2, 0.1], dtype=F64)
    row = probs.log()
    assert plain.sampling_distribution(row, 0.0, 20, 0.95).tolist() == [1, 0, 0, 0]
    assert torch.allclose(plain.sampling_distribution(row, 1.0, 0, 1.0), probs)
    assert (plain.sampling_distribution(row, 1.0, 2, 1.0) > 0).tolist() == [True, True, False, False]
    assert (plain.sampling_distribution(row, 1.0, 0, 0.6) > 0).tolist() == [True, True, False, False]
    assert (plain.sampling_distribution(row, 1.0, 0, 0.01) > 0).tolist() == [True, False, False, False]
    sharp = plain.sampling_distribution(row, 0.5, 0, 1.0)
    assert torch.allclose(sharp, probs**2 / (probs**2).sum())


def test_batched_attention_is_the_loop_form():
    # groups of 3, a window, queries that start past the first keys, keys at given positions
    q, k, v = torch.randn(9, 6, 8, dtype=F64), torch.randn(14, 2, 8, dtype=F64), torch.randn(14, 2, 8, dtype=F64)
    for window in (0, 4):
        loop = plain.causal_attention(q, k, v, torch.arange(5, 14), window=window)
        for rows in (512, 4):
            batched = plain.causal_attention_batched(q, k, v, torch.arange(5, 14), window=window, rows=rows)
            assert torch.allclose(batched, loop, atol=1e-12)
    kp = torch.arange(100, 114)
    assert torch.allclose(plain.causal_attention_batched(q, k, v, torch.arange(105, 114), k_positions=kp),
                          plain.causal_attention(q, k, v, torch.arange(105, 114), k_positions=kp), atol=1e-12)
    raw = TINY_B
    w = plain_random_weights(raw, seed=4, std=0.2, gain_std=0.2)
    ids = torch.randint(0, raw["vocab_size"], (17,)).tolist()
    assert torch.allclose(plain.logits(raw, w, ids, batched=True), plain.logits(raw, w, ids), atol=1e-10)


def _library_head(raw, w, x):
    head = w["model.embed_tokens.weight" if raw["tie_word_embeddings"] else "lm_head.weight"].to(F64)
    h = raw["hidden_size"]
    return F.linear(F.rms_norm(x, (h,), w["model.norm.weight"].to(F64), raw["rms_norm_eps"]), head)


@pytest.mark.parametrize("raw", [TINY_A, TINY_B])
def test_without_mixer_and_feed_forward_the_model_is_embedding_norm_head(raw):
    # With o_proj and down_proj zeroed every layer adds nothing: what remains is the unscaled
    # embedding, the final norm on the stream, and the head.  An embedding multiplier, a missing
    # final norm or a head bias would show.
    w = plain_random_weights(raw, seed=6, std=0.2, gain_std=0.3)
    for name in w:
        if name.endswith("o_proj.weight") or name.endswith("down_proj.weight"):
            w[name] = torch.zeros_like(w[name])
    ids = torch.randint(0, raw["vocab_size"], (9,))
    x = w["model.embed_tokens.weight"].to(F64)[ids]
    assert torch.allclose(plain.logits(raw, w, ids.tolist()), _library_head(raw, w, x), atol=1e-10)


@pytest.mark.parametrize("raw", [TINY_A, TINY_B])
def test_layer_arrangement_against_library_routines(raw):
    # The whole arrangement spelled with library routines only: x += attn(norm_in(x));
    # x += mlp(norm_post(x)), each norm read from the un-normalised stream and each sum taken on
    # it.  Post-norm, a residual taken from the normalised rows, swapped norm gains or a
    # feed-forward fed by the attention's input would each change the result by far more than 1e-9.
    raw = dict(raw)
    w = plain_random_weights(raw, seed=8, std=0.25, gain_std=0.4)
    wd = {k: v.to(F64) for k, v in w.items()}
    T, h = 10, raw["hidden_size"]
    H, KV, D = raw["num_attention_heads"], raw["num_key_value_heads"], raw["head_dim"]
    eps, theta = raw["rms_norm_eps"], raw["rope_theta"]
    ids = torch.randint(0, raw["vocab_size"], (T,))
    pos = torch.arange(T)
    x = wd["model.embed_tokens.weight"][ids]
    for i in range(raw["num_hidden_layers"]):
        p = f"model.layers.{i}."
        a = F.rms_norm(x, (h,), wd[p + "input_layernorm.weight"], eps)
        q = F.rms_norm(F.linear(a, wd[p + "self_attn.q_proj.weight"]).view(T, H, D), (D,), wd[p + "self_attn.q_norm.weight"], eps)
        k = F.rms_norm(F.linear(a, wd[p + "self_attn.k_proj.weight"]).view(T, KV, D), (D,), wd[p + "self_attn.k_norm.weight"], eps)
        v = F.linear(a, wd[p + "self_attn.v_proj.weight"]).view(T, KV, D)
        q, k = plain.rope(q, pos, theta), plain.rope(k, pos, theta)  # pinned above by vectors and complex products
        g = H // KV
        o = F.scaled_dot_product_attention(q.transpose(0, 1), k.repeat_interleave(g, 1).transpose(0, 1),
                                           v.repeat_interleave(g, 1).transpose(0, 1), is_causal=True)
        x = x + F.linear(o.transpose(0, 1).reshape(T, H * D), wd[p + "self_attn.o_proj.weight"])
        m = F.rms_norm(x, (h,), wd[p + "post_attention_layernorm.weight"], eps)
        x = x + F.linear(F.silu(F.linear(m, wd[p + "mlp.gate_proj.weight"])) * F.linear(m, wd[p + "mlp.up_proj.weight"]),
                         wd[p + "mlp.down_proj.weight"])
    assert torch.allclose(plain.logits(raw, w, ids.tolist()), _library_head(raw, w, x), atol=1e-9)


def test_one_sublayer_at_a_time_reads_the_stream_not_the_normalised_rows():
    # One layer with the attention silenced: logits = head(norm(e + mlp(norm_post(e)))).  With the
    # feed-forward silenced instead: head(norm(e + attn(norm_in(e)))) where a single token attends
    # to itself alone, so attn is o_proj(v_proj(norm_in(e))): no softmax, rotation or q/k norm enters.
    raw = dict(TINY_B, num_hidden_layers=1)
    w = plain_random_weights(raw, seed=10, std=0.25, gain_std=0.4)
    wd = {k: v.to(F64) for k, v in w.items()}
    p, h, eps = "model.layers.0.", raw["hidden_size"], raw["rms_norm_eps"]
    e = wd["model.embed_tokens.weight"][torch.tensor([7])]
    silent = dict(w)
    silent[p + "self_attn.o_proj.weight"] = torch.zeros_like(w[p + "self_attn.o_proj.weight"])
    m = F.rms_norm(e, (h,), wd[p + "post_attention_layernorm.weight"], eps)
    mlp = F.linear(F.silu(F.linear(m, wd[p + "mlp.gate_proj.weight"])) * F.linear(m, wd[p + "mlp.up_proj.weight"]),
                   wd[p + "mlp.down_proj.weight"])
    assert torch.allclose(plain.logits(raw, silent, [7]), _library_head(raw, w, e + mlp), atol=1e-10)
    silent = dict(w)
    silent[p + "mlp.down_proj.weight"] = torch.zeros_like(w[p + "mlp.down_proj.weight"])
    a = F.rms_norm(e, (h,), wd[p + "input_layernorm.weight"], eps)
    g = raw["num_attention_heads"] // raw["num_key_value_heads"]
    v = F.linear(a, wd[p + "self_attn.v_proj.weight"]).view(1, raw["num_key_value_heads"], raw["head_dim"])
    attn = F.linear(v.repeat_interleave(g, 1).reshape(1, -1), wd[p + "self_attn.o_proj.weight"])
    assert torch.allclose(plain.logits(raw, silent, [7]), _library_head(raw, w, e + attn), atol=1e-10)
