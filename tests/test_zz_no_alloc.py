"""The attention entry point that allocates nothing (`as_attn_single_query_static`, declared in
atomserve_amd/csrc/no_alloc.h) against the entry point it is a variant of, called through ctypes."""

import ctypes

import pytest
import torch

from tests import plain_kernels as pk

pytestmark = pytest.mark.gpu

P_, I_, F_ = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
TOL = {torch.float32: dict(atol=2e-5, rtol=1e-5), torch.bfloat16: dict(atol=2e-2, rtol=2e-2)}


def static_entry():
    from atomserve_amd.kernels import build

    lib = ctypes.CDLL(build.library_path("attention"))
    fn = lib.as_attn_single_query_static
    fn.argtypes = [P_, P_, P_, I_, P_, I_, P_, P_, P_, I_, P_, I_, I_, I_, I_, F_, I_, I_, I_, P_]
    fn.restype = I_
    return fn


def case(dtype, num_tokens, contexts, H, KV, D, bs, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    pages = sum(-(-c // bs) for c in contexts) + 3
    q = torch.randn((num_tokens, H, D), generator=g, device="cuda", dtype=torch.float32).to(dtype)
    k = torch.randn((pages, KV, bs, D), generator=g, device="cuda", dtype=torch.float32).to(dtype)
    v = torch.randn((pages, KV, D, bs), generator=g, device="cuda", dtype=torch.float32).to(dtype)
    width = max(-(-c // bs) for c in contexts)
    order = torch.randperm(pages, generator=torch.Generator().manual_seed(seed)).tolist()
    tables = torch.zeros((num_tokens, width), dtype=torch.int32)
    for t, c in enumerate(contexts):
        n = -(-c // bs)
        tables[t, :n] = torch.tensor([order.pop() for _ in range(n)], dtype=torch.int32)
    positions = torch.tensor([c - 1 for c in contexts], dtype=torch.int32)
    return q, k, v, tables.cuda(), positions.cuda()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_two_calls_in_a_row_match_the_entry_point_with_buffers(dtype):
    from atomserve_amd.kernels import ops

    fn = static_entry()
    stream = torch.cuda.current_stream().cuda_stream
    H, KV, D, bs, part = 12, 4, 64, 16, 256
    # the second call is smaller in every way (tokens, contexts, partitions): it finds the first
    # call's partial results in the scratch array and must not read them
    for contexts in ([1500, 700, 1, 257, 1024, 90], [300, 40]):
        n = len(contexts)
        q, k, v, tables, positions = case(dtype, n, contexts, H, KV, D, bs, seed=len(contexts))
        want = torch.empty_like(q)
        ops.attn_single_query(q, k, v, None, positions, None, tables, want, D**-0.5, 0, max(contexts),
                              part_size=part, force_generic=True)  # fmt: skip
        got = torch.full_like(q, float("nan"))
        P = -(-max(contexts) // part)
        assert P > 1
        status = fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), 0 if dtype == torch.float32 else 1, None, n,
                    positions.data_ptr(), None, tables.data_ptr(), tables.shape[1], got.data_ptr(), H, KV, D, bs,
                    D**-0.5, 0, part, P, stream)  # fmt: skip
        assert status == 0
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        # and both are the plain attention over the same pages (a fault the two entry points share would pass the line above)
        plain = pk.paged_attention(q, k, v, torch.arange(n), positions, torch.arange(n), tables, D**-0.5)
        assert torch.allclose(got.float(), plain, **TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_listed_tokens_of_rows_and_contexts_in_one_piece(dtype):
    """The other ways to call it: some tokens of a step listed in an order of the caller's, each token
    reading the block table of its row (portions of two requests), with the contexts cut into partitions
    (the scratch array) and in one piece (no scratch at all); a window on top.  Against the plain
    attention, and bit for bit against the entry point with buffers."""
    from atomserve_amd.kernels import ops

    fn = static_entry()
    stream = torch.cuda.current_stream().cuda_stream
    H, KV, D, bs = 6, 2, 32, 8
    contexts = [330, 61]  # two requests; the step brings the last 5 tokens of the first and the last 3 of the second
    q, k, v, tables, _ = case(dtype, 8, contexts, H, KV, D, bs, seed=9)
    tables = tables[:2].contiguous()
    positions = torch.tensor([325, 326, 327, 328, 329, 58, 59, 60], dtype=torch.int32, device="cuda")
    tok_row = torch.tensor([0, 0, 0, 0, 0, 1, 1, 1], dtype=torch.int32, device="cuda")
    items = torch.tensor([7, 2, 4, 5, 0], dtype=torch.int32, device="cuda")  # five of the eight, in no order
    for window, part in ((0, 64), (0, 512), (40, 64)):
        P = -(-max(contexts) // part)
        got = torch.zeros_like(q)
        status = fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), 0 if dtype == torch.float32 else 1, items.data_ptr(), 5,
                    positions.data_ptr(), tok_row.data_ptr(), tables.data_ptr(), tables.shape[1], got.data_ptr(), H, KV, D,
                    bs, D**-0.5, window, part, P, stream)  # fmt: skip
        assert status == 0 and (P == 1) == (part == 512)
        torch.cuda.synchronize()
        plain = pk.paged_attention(q, k, v, items, positions, tok_row, tables, D**-0.5, window)
        assert torch.allclose(got.float(), plain, **TOL[dtype])  # the tokens not listed stay as they were: zero
        want = torch.zeros_like(q)
        ops.attn_single_query(q, k, v, items, positions, tok_row, tables, want, D**-0.5, window, max(contexts),
                              part_size=part, force_generic=True)  # fmt: skip
        assert torch.equal(got, want)


def test_a_call_beyond_the_scratch_array_is_refused_before_any_launch():
    fn = static_entry()
    # 4096 tokens x 32 heads x 64 partitions x (128 + 2) floats is far beyond 2 Mi floats; the
    # pointers are never touched because nothing is launched
    status = fn(None, None, None, 1, None, 4096, None, None, None, 64, None, 32, 8, 128, 16, 0.1, 0, 256, 64, None)
    assert status == -4
    # without partitions no scratch is needed, so any number of tokens is taken; zero tokens is no work
    assert fn(None, None, None, 1, None, 0, None, None, None, 64, None, 32, 8, 128, 16, 0.1, 0, 256, 1, None) == 0
