"""Grouped-query softmax attention over a paged cache (the mixer of this architecture).

    qkv = h @ qkv_w^T;  q, k <- per-head norm (optional), rotation (optional)
    k, v -> cache pages at the tokens' slots, written before attending
    o = softmax(q k^T * scale over the keys a query may see) v;  out = o @ o_w^T

(reference atomserve/model.py:292-336).  Every size, the scale, the window, the norm
and the position encoding arrive through the spec.  A run that only reads another
run's cache computes q alone and stores nothing.
"""

import torch

from atomserve_amd.kernels import ops
from atomserve_amd.parts.base import Mixer, PagedCacheRequest, PendingNorm, SplitSums, WeightDecl, build, register

# Rows with at most SHORT_ROW new tokens are attended as that many single queries
# (reference atomserve/runner.py:31-34); longer rows go through the prefill kernel in work items of
# TILE_Q consecutive queries.  The step's batch sorts its rows so because this mixer asks for it.
SHORT_ROW = 8
TILE_Q = ops.PREFILL_TILE_QUERIES


class Attention(Mixer):
    takes_pending_norm = True
    adds_to_residual = True

    @property
    def capturable(self) -> bool:
        return self.position is None or self.position.capturable

    def __init__(self, spec, env):
        super().__init__(spec, env)
        s = spec
        if s.num_heads % s.num_kv_heads:
            raise ValueError(f"{s.num_heads} query heads do not divide over {s.num_kv_heads} kv heads")
        chunk = 4 if env.dtype == torch.float32 else 8
        if s.head_dim % chunk or s.head_dim > ops.SINGLE_QUERY_MAX_HEAD_DIM:
            raise ValueError(
                f"head_dim {s.head_dim} is not supported by the attention kernels "
                f"(a multiple of {chunk}, at most {ops.SINGLE_QUERY_MAX_HEAD_DIM})"
            )
        # What the kernels compute and nothing else: a per-head RMSNorm, and a rotation of the pairs
        # (i, i + R/2) of a head's first R coordinates by angles that the position part tabulates.
        if s.qk_norm is not None and s.qk_norm.kind != "rmsnorm":
            raise ValueError(f"the attention kernels norm heads by 'rmsnorm' only, not by {s.qk_norm.kind!r}")
        if s.qk_norm is not None and s.qk_norm.size != s.head_dim:
            raise ValueError(f"the per-head norm has {s.qk_norm.size} gains, a head {s.head_dim} coordinates")
        self.position = build("position", s.position, env) if s.position is not None else None
        if self.position is not None and getattr(self.position, "pairs", None) != "half":
            raise ValueError(
                f"the attention kernels rotate the pairs (i, i + R/2) by a table of cosines and sines "
                f"(a position part that declares pairs = 'half'); {s.position.kind!r} declares "
                f"{getattr(self.position, 'pairs', None)!r}"
            )
        self.q_norm_weight = self.k_norm_weight = None

    def weight_decls(self) -> dict:
        s = self.spec
        decls = {
            "qkv.weight": WeightDecl(((s.num_heads + 2 * s.num_kv_heads) * s.head_dim, s.hidden_size)),
            "o.weight": WeightDecl((s.hidden_size, s.num_heads * s.head_dim)),
        }
        if s.qk_norm is not None:
            decls["q_norm.weight"] = WeightDecl((s.head_dim,), role="vector")
            decls["k_norm.weight"] = WeightDecl((s.head_dim,), role="vector")
        return decls

    def bind(self, tensors: dict) -> None:
        super().bind(tensors)
        # what the products of a decode step stream: the matrices with their copies in wave order
        self.qkv = ops.Streamed(self.qkv_weight, self.env.stream_copies)
        self.o = ops.Streamed(self.o_weight, self.env.stream_copies)

    def streamed(self) -> list:
        return [self.qkv, self.o]

    def cache_request(self):
        s = self.spec
        return PagedCacheRequest(s.num_kv_heads, s.head_dim, s.window)

    def row_split(self):
        return (SHORT_ROW, TILE_Q)

    def forward(self, h, step, cache, residual=None, next_norm=None):
        """h [T, hidden] compute dtype (or the norm left pending on the stream) -> [T, hidden], or the
        pending `next_norm` after adding the output into `residual`.  cache: a PagedLayerView (pages
        of this run's cache, its group's slots and block tables for this step, whether to store)."""
        s, env = self.spec, self.env
        pending = isinstance(h, PendingNorm)
        T, device = (h.x.shape[0], h.x.device) if pending else (h.shape[0], h.device)
        H, KV, D = s.num_heads, s.num_kv_heads, s.head_dim
        qkv = torch.empty((T, (H + 2 * KV) * D), dtype=env.dtype, device=device)
        if pending:
            h.gemm(self.qkv, qkv)
        else:
            ops.gemm(h, self.qkv, qkv, env.products)
        cos_sin = self.position.prepare(step) if self.position is not None else None
        eps = s.qk_norm.eps if s.qk_norm is not None else 0.0
        rotary = 2 * cos_sin.shape[1] if cos_sin is not None else 0
        if step.decode_only and ops.attn_decode_fresh_supported(env.dtype, H, KV, D, cache.block_size, rotary,
                                                                s.qk_norm is not None):  # fmt: skip
            # a decode step: norm, rotation, the cache store and attention in one kernel
            out = torch.empty((T, H, D), dtype=env.dtype, device=device)
            ops.attn_decode_fresh(
                qkv.view(T, H + 2 * KV, D), self.q_norm_weight, self.k_norm_weight, cos_sin, cache.slots, eps,
                cache.writes, cache.k_pages, cache.v_pages, step.positions, cache.block_tables, out, H, s.scale,
                s.window, step.max_context, order=step.all_tokens,
            )  # fmt: skip
        else:
            q = torch.empty((T, H, D), dtype=env.dtype, device=device)
            ops.qk_norm_rope_store(
                qkv.view(T, H + 2 * KV, D), self.q_norm_weight, self.k_norm_weight, cos_sin, cache.slots, q,
                cache.k_pages, cache.v_pages, H, KV, eps, store_kv=cache.writes,
            )  # fmt: skip
            out = torch.empty((T, H, D), dtype=env.dtype, device=device)
            self.attend(q, out, step, cache)
        if residual is not None and next_norm is not None:
            link = next_norm.absorb(out.view(T, H * D), self.o, residual)
            if link is not None:
                return link
            if next_norm.takes_split_sums:
                plan = ops.gemm_split_plan(T, s.hidden_size, out.view(T, H * D).shape[1], env.dtype)
                if plan is not None:
                    return SplitSums(ops.gemm_split(out.view(T, H * D), self.o, plan))
        y = torch.empty((T, s.hidden_size), dtype=env.dtype, device=device)
        ops.gemm(out.view(T, H * D), self.o, y, env.products)
        return y

    def attend(self, q, out, step, cache) -> None:
        s = self.spec
        # fp32, and shapes the prefill kernel does not take: every token is a single query.
        # Otherwise short rows are single queries and long rows go through the prefill kernel.
        if step.decode_only:  # token t is row t: the kernels need no maps from one to the other
            ops.attn_single_query(q, cache.k_pages, cache.v_pages, step.all_tokens, step.positions, None,
                                  cache.block_tables, out, s.scale, s.window, step.max_context)  # fmt: skip
            return
        if not ops.attn_prefill_supported(self.env.dtype, s.head_dim, cache.block_size):
            ops.attn_single_query(q, cache.k_pages, cache.v_pages, step.all_tokens, step.positions, step.tok_row,
                                  cache.block_tables, out, s.scale, s.window, step.max_context)  # fmt: skip
            return
        rows = step.split(self.row_split())
        if rows.num_short_tokens:
            ops.attn_single_query(q, cache.k_pages, cache.v_pages, rows.short_tokens, step.positions, step.tok_row,
                                  cache.block_tables, out, s.scale, s.window, rows.max_short_context)  # fmt: skip
        if rows.num_long_tiles:
            ops.attn_prefill(q, cache.k_pages, cache.v_pages, rows.long_tiles, cache.block_tables, out, s.scale,
                             s.window, step.max_context, tile_keys=rows.tile_keys)  # fmt: skip


register("mixer", "attention", Attention)
