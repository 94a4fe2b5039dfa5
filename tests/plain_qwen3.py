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
    i = torch.arange(0, head_dim, 2, dtype=torch.float64, device=positions.device)
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
        k_positions = torch.arange(S, device=q.device)
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


def _same(x):
    return x


def rounder(storage_dtype):
    """x -> x rounded to `storage_dtype` and back: what an engine that keeps its activations in that
    type does to them between kernels.  None: no rounding."""
    if storage_dtype is None:
        return _same
    return lambda x: x.to(storage_dtype).to(x.dtype)


def causal_attention_batched(q, k, v, q_positions, window: int = 0, k_positions=None, rows: int = 512, rnd=_same):
    """The same function as `causal_attention` with the loops over heads and queries written as
    masked matrix products, `rows` queries at a time, for sequences and head counts at which the
    loops would take hours (tests/test_plain.py holds the two equal).  Scores of hidden keys are
    set to -inf before the softmax, which gives them weight zero exactly."""
    T, H, D = q.shape
    S, KV, _ = k.shape
    group = H // KV
    if k_positions is None:
        k_positions = torch.arange(S, device=q.device)
    out = torch.empty_like(q)
    kg, vg = k.transpose(0, 1), v.transpose(0, 1)  # [KV, S, D]
    for t0 in range(0, T, rows):
        qp = q_positions[t0 : t0 + rows]
        n = qp.shape[0]
        qq = q[t0 : t0 + n].reshape(n, KV, group, D).permute(1, 2, 0, 3)  # [KV, group, n, D]
        scores = torch.einsum("kgnd,ksd->kgns", qq, kg) / math.sqrt(D)
        seen = k_positions[None, :] <= qp[:, None]
        if window > 0:
            seen = seen & (k_positions[None, :] > qp[:, None] - window)
        scores = scores.masked_fill(~seen[None, None], float("-inf"))
        if rnd is _same:
            weights = torch.softmax(scores, dim=-1)
            o = torch.einsum("kgns,ksd->kgnd", weights, vg)
        else:  # a kernel that keeps exp(s - max) in the storage type for its second product
            e = torch.exp(scores - scores.max(dim=-1, keepdim=True).values)
            o = torch.einsum("kgns,ksd->kgnd", rnd(e), vg) / e.sum(dim=-1, keepdim=True)
        out[t0 : t0 + n] = o.permute(2, 0, 1, 3).reshape(n, H, D)
    return out


def swiglu(x: torch.Tensor, gate_w: torch.Tensor, up_w: torch.Tensor, down_w: torch.Tensor, rnd=_same):
    """down( silu(gate(x)) * up(x) ), silu(g) = g / (1 + exp(-g))
    (reference atomserve/model.py:354-360, atomserve/kernels.py:446-448)."""
    g = rnd(x @ gate_w.T)
    u = rnd(x @ up_w.T)
    return rnd(rnd((g / (1.0 + torch.exp(-g))) * u) @ down_w.T)


def attention_layer(x, w, prefix, cfg, positions, attention=causal_attention, rnd=_same):  # positions are absolute
    """(cfg["window"], if present, limits the keys a query sees; Qwen3 has none.)
    Projection, per-head RMSNorm of q and k (same eps as the layer norms, before the
    rotation, v untouched), rotation, attention, output projection
    (reference atomserve/model.py:317-336)."""
    T = x.shape[0]
    H, KV, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps, theta = cfg["rms_norm_eps"], cfg["rope_theta"]
    q = rnd(x @ w[prefix + "self_attn.q_proj.weight"].T).view(T, H, D)
    k = rnd(x @ w[prefix + "self_attn.k_proj.weight"].T).view(T, KV, D)
    v = rnd(x @ w[prefix + "self_attn.v_proj.weight"].T).view(T, KV, D)
    q = rms_norm(q, w[prefix + "self_attn.q_norm.weight"], eps)
    k = rms_norm(k, w[prefix + "self_attn.k_norm.weight"], eps)
    q, k = rnd(rope(q, positions, theta)), rnd(rope(k, positions, theta))
    extra = {} if rnd is _same else {"rnd": rnd}
    o = rnd(attention(q, k, v, positions, window=cfg.get("window", 0), k_positions=positions, **extra))
    return rnd(o.reshape(T, H * D) @ w[prefix + "self_attn.o_proj.weight"].T)


def normalise_config(raw: dict) -> dict:
    """The numbers of config.json with the reference's one default
    (head_dim = hidden/heads, reference atomserve/config.py:55)."""
    cfg = dict(raw)
    cfg.setdefault("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"])
    cfg.setdefault("tie_word_embeddings", False)
    return cfg


class _Cast:
    """A checkpoint's tensors in `dtype`, converted one at a time when asked for (a model of 8 B
    parameters is not held twice)."""

    def __init__(self, weights: dict, dtype):
        self.weights, self.dtype = weights, dtype

    def __getitem__(self, name):
        return self.weights[name].to(self.dtype)


def hidden_states(
    raw_config: dict, weights: dict, ids, dtype=torch.float64, position_offset: int = 0, batched: bool = False,
    storage=None,
) -> torch.Tensor:
    """Residual stream after the last layer, every position of one sequence
    (reference atomserve/model.py:373-382): x += attn(norm(x)); x += mlp(norm(x)).
    Runs where the weights are (CPU or GPU); `batched` picks the matrix form of the attention.
    storage: a type (torch.bfloat16) to which everything but the residual stream, the sums inside
    norms, products and the softmax is rounded between the parts, as an engine serving in that type
    does (reference atomserve/model.py:373,377 lets activations follow the embedding's type); it needs
    the matrix form of the attention.  What it changes against the exact run is how far rounding
    alone moves the logits."""
    rnd = rounder(storage)
    if rnd is not _same and not batched:
        raise ValueError("rounded activations need the matrix form of the attention")
    cfg = normalise_config(raw_config)
    w = _Cast(weights, dtype)
    device = weights["model.embed_tokens.weight"].device
    ids = torch.as_tensor(ids, dtype=torch.long, device=device)
    positions = torch.arange(len(ids), device=device) + position_offset
    eps = cfg["rms_norm_eps"]
    attention = causal_attention_batched if batched else causal_attention
    x = embed(w["model.embed_tokens.weight"], ids)
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        h = rnd(rms_norm(x, w[p + "input_layernorm.weight"], eps))
        x = x + attention_layer(h, w, p, cfg, positions, attention, rnd)
        h = rnd(rms_norm(x, w[p + "post_attention_layernorm.weight"], eps))
        x = x + swiglu(
            h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"], rnd
        )
    return x


def logits(
    raw_config: dict, weights: dict, ids, dtype=torch.float64, position_offset: int = 0, batched: bool = False,
    storage=None,
) -> torch.Tensor:
    """Logits at every position of one sequence, [len(ids), vocab]: final norm, then the
    head, which is the embedding table when tied (reference atomserve/model.py:383-412,
    atomserve/loader.py:131-138); no scaling, capping or bias."""
    cfg = normalise_config(raw_config)
    x = hidden_states(raw_config, weights, ids, dtype, position_offset, batched, storage)
    x = rounder(storage)(rms_norm(x, weights["model.norm.weight"].to(dtype), cfg["rms_norm_eps"]))
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
