"""Plain PyTorch references of each HIP kernel, one function per kernel, in fp32/fp64
on whatever device the inputs are.  They follow the kernels' contracts (documented in
atomserve_amd/kernels/ops.py) and the reference's formulas; they share no code with
the kernels."""

import math

import torch


def embed_gather(table, ids):
    return table[ids.long()].float()


def rmsnorm(x, weight, eps, delta=None, rows=None):
    """Returns (normalised rows as fp32, x + delta as fp32)."""
    v = x.double() + (delta.double() if delta is not None else 0.0)
    sel = v if rows is None else v[rows.long()]
    out = sel / torch.sqrt((sel * sel).mean(dim=-1, keepdim=True) + eps) * weight.double()
    return out.float(), v.float()


def rope_table(positions, inv_freq):
    ang = positions.double()[:, None] * inv_freq.double()[None, :]
    return torch.stack([ang.cos(), ang.sin()], dim=-1).float()


def qk_norm_rope(qkv, q_weight, k_weight, cos_sin, num_heads, num_kv_heads, eps):
    """qkv [T, H + 2 KV, D] -> (q [T, H, D], k [T, KV, D], v [T, KV, D]) in fp32:
    per-head RMSNorm (if weights), then rotation of pairs (i, i + R/2) (if cos_sin)."""
    x = qkv.double()
    q, k, v = x.split([num_heads, num_kv_heads, num_kv_heads], dim=1)

    def norm(t, w):
        if w is None:
            return t
        return t / torch.sqrt((t * t).mean(dim=-1, keepdim=True) + eps) * w.double()

    def rot(t):
        if cos_sin is None:
            return t
        half = cos_sin.shape[1]
        c, s = cos_sin[..., 0].double()[:, None, :], cos_sin[..., 1].double()[:, None, :]
        a, b, rest = t[..., :half], t[..., half : 2 * half], t[..., 2 * half :]
        return torch.cat([a * c - b * s, b * c + a * s, rest], dim=-1)

    return rot(norm(q, q_weight)).float(), rot(norm(k, k_weight)).float(), v.float()


def store_pages(k_pages, v_pages, k, v, slots):
    """Write k, v [T, KV, D] at slot = page * bs + offset (slot < 0: skip) into k_pages
    [P, KV, bs, D] and v_pages [P, KV, D, bs] (values transposed within a page)."""
    bs = k_pages.shape[2]
    for t, slot in enumerate(slots.tolist()):
        if slot < 0:
            continue
        k_pages[slot // bs, :, slot % bs, :] = k[t].to(k_pages.dtype)
        v_pages[slot // bs, :, :, slot % bs] = v[t].to(v_pages.dtype)


def gather_context(pages, table, length, transposed=False):
    """Keys (or, transposed, values) of positions 0..length-1 of one request: [length, KV, D]."""
    bs = pages.shape[3] if transposed else pages.shape[2]
    idx = torch.arange(length, device=pages.device)
    page = torch.as_tensor(table, device=pages.device).long()[idx // bs]
    if transposed:
        return pages[page, :, :, idx % bs]
    return pages[page, :, idx % bs, :]


def paged_attention(q, k_pages, v_pages, items, positions, tok_row, block_tables, scale, window=0):
    """Single-query attention of the tokens `items` over the paged cache; returns fp32 [T, H, D]
    with the rows of other tokens left zero."""
    T, H, D = q.shape
    KV = k_pages.shape[1]
    group = H // KV
    out = torch.zeros((T, H, D), dtype=torch.float32, device=q.device)
    for t in items.tolist():
        p = int(positions[t])
        table = block_tables[int(tok_row[t])]
        k = gather_context(k_pages, table, p + 1).double()
        v = gather_context(v_pages, table, p + 1, transposed=True).double()
        lo = max(0, p - window + 1) if window > 0 else 0
        for h in range(H):
            s = (k[lo:, h // group, :] @ q[t, h].double()) * scale
            w = torch.softmax(s, dim=0)
            out[t, h] = (w @ v[lo:, h // group, :]).float()
    return out


def silu_mul(gate_up):
    g, u = gate_up.double().chunk(2, dim=-1)
    return (g / (1.0 + torch.exp(-g)) * u).float()


def gemm(a, w):
    return (a.double() @ w.double().T).float()


def topk_values(logits, k):
    return torch.topk(logits, k, dim=-1).values


def exp1_noise_bounds():
    return 1e-10, -math.log(0.5 / 16777216.0)
