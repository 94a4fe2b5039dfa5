"""The attention entry point that allocates nothing (`as_attn_single_query_static`, declared in
atomserve_amd/csrc/no_alloc.h) against the entry point it is a variant of, called through ctypes."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

P_, I_, F_ = ctypes.c_void_p, ctypes.c_int, ctypes.c_float


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


def test_a_call_beyond_the_scratch_array_is_refused_before_any_launch():
    fn = static_entry()
    # 4096 tokens x 32 heads x 64 partitions x (128 + 2) floats is far beyond 2 Mi floats; the
    # pointers are never touched because nothing is launched
    status = fn(None, None, None, 1, None, 4096, None, None, None, 64, None, 32, 8, 128, 16, 0.1, 0, 256, 64, None)
    assert status == -4
    # without partitions no scratch is needed, so any number of tokens is taken; zero tokens is no work
    assert fn(None, None, None, 1, None, 0, None, None, None, 64, None, 32, 8, 128, 16, 0.1, 0, 256, 1, None) == 0
