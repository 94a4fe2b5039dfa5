"""Which kernel, and cut how, for which sizes: the decisions of `kernels/ops.py` that need no GPU.  They
decide speed only (every route gives the same result within rounding, which the GPU tests hold them to); the
vectors here pin what the sizes say on an MI355X's 256 compute units, so that a change of a limit or a cost
shows as a change of a choice."""

import pytest
import torch

from atomserve_amd.kernels import ops

BF16, F32 = torch.bfloat16, torch.float32


@pytest.fixture(autouse=True)
def on_256_compute_units(monkeypatch):
    monkeypatch.setattr(ops, "_compute_units", 256)
    ops._prefill_plan_of.cache_clear()


def test_how_a_prompt_steps_attention_is_cut():
    """A portion behind a long prefix is few long items: cut along the keys, into the more pieces the fewer the
    items, a wave owning 32 queries where that still fills the GPU and 16 where only that does.  A lone prompt, a
    short context, a window that keeps every item short: not cut."""
    plan = lambda tokens, H, context, **kw: ops._prefill_plan(-(-tokens // 64), H, 8, 128, context, **kw)
    assert plan(512, 32, 16384) == (2, 4, 64)  # 128 items of 256 rounds: four pieces of 64 fill the 512 places
    assert plan(1024, 32, 16384) == (2, 2, 128)
    assert plan(512, 16, 16384) == (2, 8, 32)  # half the heads: twice the pieces
    assert plan(64, 32, 20000) == (1, 8, 40)  # one tile: 16 queries to a wave make twice the workgroups
    assert plan(512, 32, 4096) == (1, 2, 32)
    for tokens in (256, 512, 1024, 2048, 4096, 8192, 16384):  # lone prompts: whole
        assert plan(tokens, 32, tokens)[1:] == (1, 0) and plan(tokens, 16, tokens)[1:] == (1, 0)
    assert plan(1024, 32, 1024)[0] == 1 and plan(8192, 32, 8192)[0] == 2
    assert plan(512, 32, 1024)[1:] == (1, 0)  # 16 rounds: too short to pay for the merge
    assert plan(512, 32, 8192, window=512)[1:] == (1, 0)
    # as many items as places: whole if all are as long as the longest, cut if most are short
    assert plan(2048, 32, 16384, tile_keys=32 * 16384)[1] == 1 and plan(2048, 32, 16384, tile_keys=32 * 4000)[1] > 1
    # whatever is chosen, the pieces cover the longest item and have at least the rounds the kernel asks for
    for tokens, H, context in ((64, 8, 700), (512, 64, 40000), (130, 40, 9000), (4096, 16, 4096), (64, 32, 128)):
        for forced in (None, 2, 3, 5, 8):
            ops.PREFILL_PIECES = forced
            try:
                kind, pieces, piece_rounds = plan(tokens, H, context)
            finally:
                ops.PREFILL_PIECES = None
            rounds = -(-context // 64)
            assert kind in (1, 2) and 1 <= pieces <= 8
            assert (pieces, piece_rounds) == (1, 0) or (piece_rounds >= 2 and pieces * piece_rounds >= rounds)


def test_how_single_queries_contexts_are_partitioned():
    """Few requests: partitions of a size by which the GPU's places are filled and the merge stays small; from
    one and a half (token, kv head) pairs per compute unit on, whole contexts."""
    assert ops.attn_fill_groups() == 384
    best = lambda groups, span: min(ops.MFMA_PARTITIONS, key=lambda part: ops._partition_cost(groups, span, part))
    assert [best(8, 2048), best(64, 2048), best(64, 500)] == [256, 256, 128]
    assert [best(8, 16384), best(64, 16384), best(8, 33000)] == [512, 2048, 1024]
    # through `_partitions`, on the CPU: sizes and buffers
    size, P, m, l, acc = ops._partitions(8, 32, 8, 128, 2048, 0, True, None, "cpu")
    assert (size, P) == (256, 8) and m.shape == (8, 32, 8) and acc.shape == (8, 32, 8, 128)
    size, P, m, l, acc = ops._partitions(64, 32, 8, 128, 2100, 0, True, None, "cpu")
    assert (size, P, m) == (2112, 1, None)  # 512 pairs: the whole context, rounded up to steps of 32 keys
    size, P, *_ = ops._partitions(8, 32, 8, 128, 5000, 1024, True, None, "cpu")
    assert size == 128 and P == 40  # a window: the span decides the size, the context how many there are
    with pytest.raises(ops.KernelError, match="multiples of 32"):
        ops._partitions(8, 32, 8, 128, 2048, 0, True, 100, "cpu")


def test_how_products_of_17_to_128_rows_are_tiled():
    """Tiles of 64 weight rows, K cut into as many ranges of whole chunks as fill the compute units; the gated
    product's tile width by what the longest path loads."""
    assert ops.gemm_split_plan(64, 4096, 4096, BF16) == (4, 4)
    assert ops.gemm_split_plan(64, 4096, 12288, BF16) == (4, 4)
    assert ops.gemm_split_plan(32, 1024, 3072, BF16) == (4, 12)
    assert ops.gemm_split_plan(128, 5120, 25600, BF16) == (4, 3)
    assert ops.gemm_split_plan(8, 4096, 4096, BF16) is None  # few rows: the few-rows kernels'
    assert ops.gemm_split_plan(64, 4096, 4000, BF16) is None  # K in chunks of 256
    assert ops.gemm_split_plan(64, 4096, 4096, F32) is None
    assert [ops._gated_tile_strips(*case) for case in ((64, 12288), (64, 3072), (128, 25600))] == [6, 2, 8]
