"""A plain, slow Qwen3 decoder: whole sequences, no cache, one function per part.

Written from the formulas of the reference (aneesh-sathe/atomserve), which is read
and never run.  It shares no code with the package under test: it parses the raw
config.json dictionary itself and takes weights as a dictionary of checkpoint
tensor names.  Everything is computed in float64 by default, so that it is the
more exact side of every comparison.
"""

import math

import torch


def embed(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """Row lookup, no scaling and no position term (reference atomserve/model.py:373)."""
    return table[ids]


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """weight * x / sqrt(mean(x^2) + eps); the weight multiplies directly, no mean is
    subtracted (reference atomserve/model.py:125-139)."""
    mean_square = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return x / torch.sqrt(mean_square + eps) * weight


def rope_angles(positions: torch.Tensor, head_dim: int, theta: float) -> torch.Tensor:
    """angle[t, i] = position[t] * theta^(-2i/head_dim), i < head_dim/2
    (reference atomserve/model.py:142-148, 164)."""
    i = torch.arange(0, head_dim, 2, dtype=torch.float64)
    inv_freq = 1.0 / (float(theta) ** (i / head_dim))
    return positions.to(torch.float64)[:, None] * inv_freq[None, :]


def rope(x: torch.Tensor, positions: torch.Tensor, theta: float) -> torch.Tensor:
    """Rotate pairs (x[i], x[i + D/2]) by the token's angle: (a cos - b sin, b cos + a sin)
    (reference atomserve/model.py:172-185).  x: [T, heads, D]."""
    d = x.shape[-1]
    ang = rope_angles(positions, d, theta).to(x.dtype)  # [T, D/2]
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    a, b = x[..., : d // 2], x[..., d // 2 :]
    return torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)


def causal_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    q_positions: torch.Tensor,
    window: int = 0,
    k_positions: torch.Tensor | None = None,
) -> torch.Tensor:
    """Softmax attention of queries at absolute positions over keys (at 0..S-1 unless given).

    q [T, H, D]; k, v [S, KV, D]; query head h reads kv head h // (H/KV); a key at
    position j is seen by a query at position p iff j <= p; scale 1/sqrt(D)
    (reference atomserve/model.py:199-232, tests/test_model_unit.py:55-64).
    `window` > 0 additionally hides keys with j <= p - window (not used by Qwen3).
    """
    T, H, D = q.shape
    S, KV, _ = k.shape
    group = H // KV
    if k_positions is None:
        k_positions = torch.arange(S)
    out = torch.zeros_like(q)
    for h in range(H):
        kh, vh = k[:, h // group, :], v[:, h // group, :]
        for t in range(T):
            p = int(q_positions[t])
            seen = k_positions <= p
            if window > 0:
                seen = seen & (k_positions > p - window)
            scores = (kh[seen] @ q[t, h]) / math.sqrt(D)
            weights = torch.softmax(scores, dim=0)
            out[t, h] = weights @ vh[seen]
    return out


def swiglu(x: torch.Tensor, gate_w: torch.Tensor, up_w: torch.Tensor, down_w: torch.Tensor):
    """down( silu(gate(x)) * up(x) ), silu(g) = g / (1 + exp(-g))
    (reference atomserve/model.py:354-360, atomserve/kernels.py:446-448)."""
    g = x @ gate_w.T
    u = x @ up_w.T
    return ((g / (1.0 + torch.exp(-g))) * u) @ down_w.T


def attention_layer(x, w, prefix, cfg, positions):  # positions are absolute
    """(cfg["window"], if present, limits the keys a query sees; Qwen3 has none.)
    Projection, per-head RMSNorm of q and k (same eps as the layer norms, before the
    rotation, v untouched), rotation, attention, output projection
    (reference atomserve/model.py:317-336)."""
    T = x.shape[0]
    H, KV, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps, theta = cfg["rms_norm_eps"], cfg["rope_theta"]
    q = (x @ w[prefix + "self_attn.q_proj.weight"].T).view(T, H, D)
    k = (x @ w[prefix + "self_attn.k_proj.weight"].T).view(T, KV, D)
    v = (x @ w[prefix + "self_attn.v_proj.weight"].T).view(T, KV, D)
    q = rms_norm(q, w[prefix + "self_attn.q_norm.weight"], eps)
    k = rms_norm(k, w[prefix + "self_attn.k_norm.weight"], eps)
    q, k = rope(q, positions, theta), rope(k, positions, theta)
    o = causal_attention(q, k, v, positions, window=cfg.get("window", 0), k_positions=positions)
    return o.reshape(T, H * D) @ w[prefix + "self_attn.o_proj.weight"].T


def normalise_config(raw: dict) -> dict:
    """The numbers of config.json with the reference's one default
    (head_dim = hidden/heads, reference atomserve/config.py:55)."""
    cfg = dict(raw)
    cfg.setdefault("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"])
    cfg.setdefault("tie_word_embeddings", False)
    return cfg


def hidden_states(
    raw_config: dict, weights: dict, ids, dtype=torch.float64, position_offset: int = 0
) -> torch.Tensor:
    """Residual stream after the last layer, every position of one sequence
    (reference atomserve/model.py:373-382): x += attn(norm(x)); x += mlp(norm(x))."""
    cfg = normalise_config(raw_config)
    w = {name: t.to(dtype) for name, t in weights.items()}
    ids = torch.as_tensor(ids, dtype=torch.long)
    positions = torch.arange(len(ids)) + position_offset
    eps = cfg["rms_norm_eps"]
    x = embed(w["model.embed_tokens.weight"], ids)
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        h = rms_norm(x, w[p + "input_layernorm.weight"], eps)
        x = x + attention_layer(h, w, p, cfg, positions)
        h = rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
        x = x + swiglu(
            h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"]
        )
    return x


def logits(
    raw_config: dict, weights: dict, ids, dtype=torch.float64, position_offset: int = 0
) -> torch.Tensor:
    """Logits at every position of one sequence, [len(ids), vocab]: final norm, then the
    head, which is the embedding table when tied (reference atomserve/model.py:383-412,
    atomserve/loader.py:131-138); no scaling, capping or bias."""
    cfg = normalise_config(raw_config)
    x = hidden_states(raw_config, weights, ids, dtype, position_offset)
    x = rms_norm(x, weights["model.norm.weight"].to(dtype), cfg["rms_norm_eps"])
    head = "model.embed_tokens.weight" if cfg["tie_word_embeddings"] else "lm_head.weight"
    return x @ weights[head].to(dtype).T


def greedy(raw_config: dict, weights: dict, prompt, num_tokens: int, dtype=torch.float64):
    """Greedy continuation by recomputing the whole sequence for every token."""
    ids = list(prompt)
    for _ in range(num_tokens):
        ids.append(int(logits(raw_config, weights, ids, dtype)[-1].argmax()))
    return ids[len(prompt) :]


# ---- sampling (reference atomserve/sampler.py:82-129) ---------------------------------


def sampling_distribution(row: torch.Tensor, temperature: float, top_k: int, top_p: float):
    """The distribution the reference samples from, dense over the vocabulary.

    top-k on the raw logits (0 or >= vocab disables), divide by the temperature,
    softmax, then drop a token once the mass ranked above it reaches top_p; the best
    token always survives (reference atomserve/sampler.py:91-117).  Temperature 0 is
    the argmax.  Returned unnormalised after top-p, as the exponential race uses it.
    """
    row = row.to(torch.float64)
    vocab = row.shape[0]
    if temperature == 0:
        out = torch.zeros(vocab, dtype=torch.float64)
        out[int(row.argmax())] = 1.0
        return out
    k = top_k if 0 < top_k < vocab else vocab
    values, indices = torch.sort(row, descending=True, stable=True)
    values, indices = values[:k], indices[:k]
    probs = torch.softmax(values / temperature, dim=0)
    mass_before = torch.cumsum(probs, dim=0) - probs
    probs = torch.where(mass_before >= top_p, torch.zeros_like(probs), probs)
    out = torch.zeros(vocab, dtype=torch.float64)
    out[indices] = probs
    return out
