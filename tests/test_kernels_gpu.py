"""Each HIP kernel alone against its plain reference (tests/plain_kernels.py), at sizes
other than the tiny models'.  fp32 differences are real faults; bf16 results may differ
from the rounded reference by one rounding step."""

import math

import pytest
import torch

from tests import plain_kernels as pk

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32, BF16, I32 = torch.float32, torch.bfloat16, torch.int32


@pytest.fixture(scope="module")
def ops():
    from atomserve_amd.kernels import ops as module

    return module


def close_bf16(got, ref, scale=None):
    """Equal to the reference rounded to bfloat16, up to one step of the larger magnitude."""
    got, ref = got.float(), ref.float()
    step = torch.maximum(ref.abs(), got.abs()) * 2.0**-7 + (1e-6 if scale is None else scale * 2.0**-8)
    return bool(((got - ref).abs() <= step).all())


def i32(values):
    return torch.tensor(values, dtype=I32, device=DEV)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_embed_gather(ops, dtype):
    torch.manual_seed(0)
    table = torch.randn(1000, 96, device=DEV).to(dtype)
    ids = i32([0, 999, 5, 5, 731, 12, 1])
    out = torch.full((7, 96), 7.0, device=DEV)
    ops.embed_gather(table, ids, out)
    assert torch.equal(out, pk.embed_gather(table, ids))


@pytest.mark.parametrize("n", [96, 97, 1000, 4096, 5120, 20000])
@pytest.mark.parametrize("rows", [1, 7, 300])
def test_rmsnorm_fp32(ops, n, rows):
    torch.manual_seed(1)
    x = torch.randn(rows, n, device=DEV) * 3
    w = torch.randn(n, device=DEV) + 1
    out = torch.empty_like(x)
    ops.rmsnorm(x, w, 1e-5, out)
    ref, _ = pk.rmsnorm(x, w, 1e-5)
    assert torch.allclose(out, ref, atol=1e-5, rtol=1e-6)


@pytest.mark.parametrize("out_dtype,w_dtype", [(F32, F32), (BF16, BF16), (BF16, F32)])
def test_rmsnorm_adds_the_pending_delta_and_selects_rows(ops, out_dtype, w_dtype):
    torch.manual_seed(2)
    T, n = 37, 200
    x0 = torch.randn(T, n, device=DEV) * 2
    delta = torch.randn(T, n, device=DEV).to(out_dtype)
    w = (torch.randn(n, device=DEV) * 0.2 + 1).to(w_dtype)
    # fused sum, written back
    x = x0.clone()
    out = torch.empty(T, n, dtype=out_dtype, device=DEV)
    ops.rmsnorm(x, w, 1e-6, out, delta=delta)
    ref, new_x = pk.rmsnorm(x0, w, 1e-6, delta)
    assert torch.allclose(x, new_x, atol=1e-6)
    assert torch.allclose(out.float(), ref, atol=1e-5) if out_dtype == F32 else close_bf16(out, ref)
    # row selection without touching x
    rows = i32([36, 0, 5, 5])
    x = x0.clone()
    out = torch.empty(4, n, dtype=out_dtype, device=DEV)
    ops.rmsnorm(x, w, 1e-6, out, delta=delta, rows=rows, update_x=False)
    ref, _ = pk.rmsnorm(x0, w, 1e-6, delta, rows)
    assert torch.equal(x, x0)
    assert torch.allclose(out.float(), ref, atol=1e-5) if out_dtype == F32 else close_bf16(out, ref)


def test_rmsnorm_eps_matters(ops):
    x = torch.full((1, 64), 1e-3, device=DEV)
    w = torch.ones(64, device=DEV)
    a, b = torch.empty_like(x), torch.empty_like(x)
    ops.rmsnorm(x, w, 1e-6, a)
    ops.rmsnorm(x, w, 1e-2, b)
    assert torch.allclose(a, torch.full_like(a, 1e-3 / math.sqrt(2e-6)), rtol=1e-5)
    assert torch.allclose(b, torch.full_like(b, 1e-3 / math.sqrt(1e-6 + 1e-2)), rtol=1e-5)


def test_rope_table_large_positions(ops):
    # positions from reference tests/test_kernels.py:35, theta 1e6
    pos = i32([0, 1, 300, 4097, 39999])
    inv = (1.0 / (1e6 ** (torch.arange(0, 128, 2, dtype=torch.float64) / 128))).to(DEV)
    out = torch.empty(5, 64, 2, device=DEV)
    ops.rope_table(pos, inv, out)
    assert torch.allclose(out, pk.rope_table(pos, inv), atol=2e-7, rtol=0)
    assert torch.equal(out[0, :, 0], torch.ones(64, device=DEV)) and torch.equal(out[0, :, 1], torch.zeros(64, device=DEV))


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("heads,D,bs", [((16, 8), 128, 16), ((32, 8), 128, 16), ((6, 2), 32, 8), ((5, 5), 48, 4), ((4, 1), 16, 16)])
def test_qk_norm_rope_store(ops, dtype, heads, D, bs):
    H, KV = heads
    torch.manual_seed(3)
    pos = i32([0, 1, 300, 4097, 39999])
    slots = i32([3, 9, 17, 2, 30])
    qkv = (torch.randn(5, H + 2 * KV, D, device=DEV) * 3).to(dtype)
    qw, kw = (torch.randn(D, device=DEV) + 1).to(dtype), (torch.randn(D, device=DEV) + 1).to(dtype)
    inv = (1.0 / (1e6 ** (torch.arange(0, D, 2, dtype=torch.float64) / D))).to(DEV)
    cs = torch.empty(5, D // 2, 2, device=DEV)
    ops.rope_table(pos, inv, cs)
    pages = 64 // bs
    k_pages = torch.zeros(pages, KV, bs, D, dtype=dtype, device=DEV)
    v_pages = torch.zeros(pages, KV, D, bs, dtype=dtype, device=DEV)
    q = torch.empty(5, H, D, dtype=dtype, device=DEV)
    ops.qk_norm_rope_store(qkv, qw, kw, cs, slots, q, k_pages, v_pages, H, KV, 1e-6)
    rq, rk, rv = pk.qk_norm_rope(qkv, qw, kw, cs, H, KV, 1e-6)
    ref_k, ref_v = torch.zeros(pages, KV, bs, D, device=DEV), torch.zeros(pages, KV, D, bs, device=DEV)
    pk.store_pages(ref_k, ref_v, rk, rv, slots)
    if dtype == F32:
        assert torch.allclose(q, rq, atol=1e-5) and torch.allclose(k_pages, ref_k, atol=1e-5)
    else:
        assert close_bf16(q, rq) and close_bf16(k_pages, ref_k)
    assert torch.equal(v_pages.float(), ref_v)  # values are copied bit for bit; untouched slots stay zero
    assert (k_pages.float().abs().sum(dim=(1, 3)) > 0).sum() == 5


@pytest.mark.parametrize("D,bs,gain,rope", [(128, 16, BF16, True), (64, 32, F32, True), (256, 16, BF16, True),
                                              (128, 16, None, True), (32, 16, F32, False)])
def test_qk_norm_rope_store_many_tokens_bf16(ops, D, bs, gain, rope):
    """A prompt's worth of rows through the 16-byte path: fp32 or bf16 gains, no norm, no rotation,
    tokens whose keys are not stored, q alone."""
    H, KV, T = 6, 2, 333
    torch.manual_seed(13)
    qkv = (torch.randn(T, H + 2 * KV, D, device=DEV) * 3).to(BF16)
    qw = kw = None
    if gain is not None:
        qw, kw = (torch.randn(D, device=DEV) + 1).to(gain), (torch.randn(D, device=DEV) + 1).to(gain)
    cs = None
    if rope:
        inv = (1.0 / (1e6 ** (torch.arange(0, D, 2, dtype=torch.float64) / D))).to(DEV)
        cs = torch.empty(T, D // 2, 2, device=DEV)
        ops.rope_table(i32(list(range(1000, 1000 + T))), inv, cs)
    pages = -(-T // bs) + 1
    perm = torch.randperm(pages * bs)[:T].tolist()
    perm[7] = perm[100] = -1
    slots = i32(perm)
    k_pages = torch.zeros(pages, KV, bs, D, dtype=BF16, device=DEV)
    v_pages = torch.zeros(pages, KV, D, bs, dtype=BF16, device=DEV)
    q = torch.empty(T, H, D, dtype=BF16, device=DEV)
    ops.qk_norm_rope_store(qkv, qw, kw, cs, slots, q, k_pages, v_pages, H, KV, 1e-6)
    rq, rk, rv = pk.qk_norm_rope(qkv, qw, kw, cs, H, KV, 1e-6)
    ref_k, ref_v = torch.zeros(pages, KV, bs, D, device=DEV), torch.zeros(pages, KV, D, bs, device=DEV)
    keep = [i for i, sl in enumerate(perm) if sl >= 0]
    pk.store_pages(ref_k, ref_v, rk[keep], rv[keep], i32([perm[i] for i in keep]))
    assert close_bf16(q, rq) and close_bf16(k_pages, ref_k)
    assert torch.equal(v_pages.float(), ref_v)
    q2 = torch.empty_like(q)
    ops.qk_norm_rope_store(qkv, qw, kw, cs, None, q2, None, None, H, KV, 1e-6, store_kv=False)
    assert torch.equal(q2, q)
    # a prompt's own layout: slots that follow one another from the middle of a page on
    run = list(range(5, 5 + T))
    k_run, v_run = torch.zeros_like(k_pages), torch.zeros_like(v_pages)
    ops.qk_norm_rope_store(qkv, qw, kw, cs, i32(run), q2, k_run, v_run, H, KV, 1e-6)
    ref_k.zero_(), ref_v.zero_()
    pk.store_pages(ref_k, ref_v, rk, rv, i32(run))
    assert close_bf16(k_run, ref_k) and torch.equal(v_run.float(), ref_v)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_what_is_not_finite_never_reaches_the_cache(ops, dtype):
    """A model that overflows hands the store kernels infinities and NaNs.  Pages are used again by
    other requests, and kernels multiply masked places by zero, so the pools hold finite values
    only: what is not finite is stored as zero; finite values and the queries are untouched."""
    H, KV, D, bs = 4, 2, 64, 16
    torch.manual_seed(17)
    qkv = torch.randn(40, H + 2 * KV, D, device=DEV).to(dtype)
    bad = qkv.clone()
    bad[3, H, 5] = float("inf")  # a key
    bad[7, H + KV + 1, 9] = float("nan")  # a value
    bad[20, H + KV, 0] = float("-inf")  # another value
    bad[11, H + 1, 63] = 3.0e38 if dtype == BF16 else float("inf")  # finite, and stays so after the norm
    qw, kw = torch.ones(D, device=DEV, dtype=dtype), torch.ones(D, device=DEV, dtype=dtype)
    inv = (1.0 / (1e4 ** (torch.arange(0, D, 2, dtype=torch.float64) / D))).to(DEV)
    cs = torch.empty(40, D // 2, 2, device=DEV)
    ops.rope_table(i32(list(range(40))), inv, cs)
    slots = i32(list(range(8, 48)))
    for weights in ((qw, kw), (None, None)):
        k_pages = torch.zeros(4, KV, bs, D, dtype=dtype, device=DEV)
        v_pages = torch.zeros(4, KV, D, bs, dtype=dtype, device=DEV)
        q = torch.empty(40, H, D, dtype=dtype, device=DEV)
        ops.qk_norm_rope_store(bad, *weights, cs, slots, q, k_pages, v_pages, H, KV, 1e-6)
        assert torch.isfinite(k_pages).all() and torch.isfinite(v_pages).all()
        good_k, good_v, good_q = torch.zeros_like(k_pages), torch.zeros_like(v_pages), torch.empty_like(q)
        ops.qk_norm_rope_store(qkv, *weights, cs, slots, good_q, good_k, good_v, H, KV, 1e-6)
        assert torch.equal(q, good_q)
        clean = torch.ones(40, dtype=torch.bool, device=DEV)
        clean[[3, 7, 20, 11]] = False
        rows_k = k_pages.permute(0, 2, 1, 3).reshape(-1, KV, D)[8:48]
        rows_v = v_pages.permute(0, 3, 1, 2).reshape(-1, KV, D)[8:48]
        assert torch.equal(rows_k[clean], good_k.permute(0, 2, 1, 3).reshape(-1, KV, D)[8:48][clean])
        assert torch.equal(rows_v[clean], good_v.permute(0, 3, 1, 2).reshape(-1, KV, D)[8:48][clean])
        assert rows_v[7, 1, 9] == 0 and rows_v[20, 0, 0] == 0


def test_a_decode_step_keeps_the_cache_finite_too(ops):
    H, KV, D, bs = 8, 2, 128, 16
    lens = [5, 40, 300]
    _, k_pages, v_pages, tables, positions = paged_case(BF16, H, KV, D, bs, lens, seed=3)
    qkv = torch.randn(3, H + 2 * KV, D, device=DEV).to(BF16)
    qkv[1, H + KV, 7] = float("nan")  # a value of the new token
    qkv[2, H + 1, 3] = float("inf")  # a coordinate of its key: the norm makes the whole key NaN
    g = torch.ones(D, device=DEV, dtype=BF16)
    inv = (1.0 / (1e4 ** (torch.arange(0, D, 2, dtype=torch.float64) / D))).to(DEV)
    cs = torch.empty(3, D // 2, 2, device=DEV)
    ops.rope_table(positions, inv, cs)
    slots = i32([tables[i, (n - 1) // bs].item() * bs + (n - 1) % bs for i, n in enumerate(lens)])
    out = torch.zeros(3, H, D, dtype=BF16, device=DEV)
    ops.attn_decode_fresh(qkv, g, g, cs, slots, 1e-6, True, k_pages, v_pages, positions, tables, out, H, D**-0.5, 0, max(lens))
    torch.cuda.synchronize()
    assert torch.isfinite(k_pages).all() and torch.isfinite(v_pages).all() and torch.isfinite(out[0]).all()


def test_wide_heads_in_large_groups_go_to_the_general_kernel(ops):
    """16 heads of 256 to one kv head would need more LDS than a workgroup of the matrix-core decode
    kernel gets: such shapes are routed to the general kernel (test_attention_single_query runs them)
    and the one-kernel decode step is not offered for them."""
    assert not ops.attn_decode_fresh_supported(BF16, 16, 1, 256, 16, 256, True)
    assert ops.attn_decode_fresh_supported(BF16, 16, 2, 256, 16, 256, True)
    assert ops.attn_decode_fresh_supported(BF16, 16, 1, 128, 16, 128, True)


def test_qk_norm_rope_store_variants(ops):
    """No norm, no rotation, a rotation of part of the head, and q alone (a run that reads
    another run's cache stores nothing)."""
    torch.manual_seed(4)
    H, KV, D = 4, 2, 32
    qkv = torch.randn(3, H + 2 * KV, D, device=DEV)
    pos, slots = i32([5, 6, 7]), i32([0, -1, 9])
    inv = (1.0 / (1e4 ** (torch.arange(0, 16, 2, dtype=torch.float64) / 16))).to(DEV)
    cs = torch.empty(3, 8, 2, device=DEV)
    ops.rope_table(pos, inv, cs)
    k_pages, v_pages = torch.zeros(2, KV, 8, D, device=DEV), torch.zeros(2, KV, D, 8, device=DEV)
    q = torch.empty(3, H, D, device=DEV)
    ops.qk_norm_rope_store(qkv, None, None, cs, slots, q, k_pages, v_pages, H, KV, 0.0)
    rq, rk, rv = pk.qk_norm_rope(qkv, None, None, cs, H, KV, 0.0)
    assert torch.allclose(q, rq, atol=1e-6)
    assert torch.equal(q[..., 16:], qkv[:, :H, 16:])  # beyond the rotary width nothing changes
    assert torch.allclose(k_pages[0, :, 0], rk[0], atol=1e-6) and torch.allclose(k_pages[1, :, 1], rk[2], atol=1e-6)
    assert k_pages.abs().sum(dim=(1, 3)).count_nonzero() == 2  # the token with slot -1 stored nothing
    q2 = torch.empty_like(q)
    ops.qk_norm_rope_store(qkv, None, None, None, None, q2, None, None, H, KV, 0.0, store_kv=False)
    assert torch.equal(q2, qkv[:, :H])


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("rows,inter", [(1, 3072), (7, 3072), (300, 3072), (5, 160), (33, 100), (2048, 1536)])
def test_silu_mul(ops, dtype, rows, inter):
    # sizes from reference tests/test_kernels.py:192-198
    torch.manual_seed(5)
    gu = (torch.randn(rows, 2 * inter, device=DEV) * 3).to(dtype)
    out = torch.empty(rows, inter, dtype=dtype, device=DEV)
    ops.silu_mul(gu, out)
    ref = pk.silu_mul(gu)
    assert torch.allclose(out, ref, atol=1e-5) if dtype == F32 else close_bf16(out, ref)


@pytest.mark.parametrize("M,N,K", [(1, 96, 64), (7, 1000, 96), (130, 257, 193), (64, 64, 16), (65, 63, 17), (3, 2000, 4096)])
def test_gemm_fp32_is_true_fp32(ops, M, N, K):
    torch.manual_seed(6)
    a, w = torch.randn(M, K, device=DEV), torch.randn(N, K, device=DEV)
    out = torch.empty(M, N, device=DEV)
    ops.gemm(a, w, out)
    ref = pk.gemm(a, w)
    assert torch.allclose(out, ref, atol=2e-6 * math.sqrt(K) * 4, rtol=1e-6)
    # a reduced-precision matrix mode (bf16 or tf32-like inputs) would be off by about 1e-3 * sqrt(K)
    assert (out - ref).abs().max() < 1e-4 * math.sqrt(K)


def test_gemm_fp32_rows_do_not_depend_on_the_batch(ops):
    torch.manual_seed(7)
    a, w = torch.randn(70, 200, device=DEV), torch.randn(300, 200, device=DEV)
    full = torch.empty(70, 300, device=DEV)
    ops.gemm(a, w, full)
    for i in (0, 63, 64, 69):
        one = torch.empty(1, 300, device=DEV)
        ops.gemm(a[i : i + 1].contiguous(), w, one)
        assert torch.equal(one[0], full[i])


@pytest.mark.parametrize("M,N,K", [(1, 96, 64), (8, 1000, 96), (64, 4096, 1024), (300, 257, 192), (5, 2000, 4096),
                                   (16, 4096, 4096), (12, 8200, 4096), (9, 16000, 2048), (3, 40, 200), (16, 24, 8),
                                   (4, 1040, 5120), (7, 520, 6144), (2, 100, 2560), (11, 4100, 3072), (8, 512, 12288),
                                   (13, 300, 6152), (17, 300, 4096), (32, 6144, 1024), (25, 1000, 1000),
                                   (31, 520, 3072), (20, 64, 4096), (32, 300, 24), (32, 6144, 4096), (8, 6150, 4096), (1, 10240, 2048),
                                   (24, 6147, 1024), (9, 304, 2304), (16, 6144, 2560), (20, 96, 2560)])  # fmt: skip
def test_gemm_bf16(ops, M, N, K):
    torch.manual_seed(8)
    a, w = torch.randn(M, K, device=DEV).to(BF16), torch.randn(N, K, device=DEV).to(BF16)
    ref = pk.gemm(a, w)
    out = torch.empty(M, N, dtype=BF16, device=DEV)
    ops.gemm(a, w, out)
    assert close_bf16(out, ref, scale=math.sqrt(K))
    out32 = torch.empty(M, N, dtype=F32, device=DEV)
    ops.gemm(a, w, out32)
    assert torch.allclose(out32, ref, atol=math.sqrt(K) * 2.0**-8, rtol=2.0**-7)


@pytest.mark.parametrize("M,I,K", [(1, 96, 64), (8, 1000, 96), (5, 1030, 4096), (16, 12288, 4096), (9, 700, 2048),
                                   (3, 40, 200), (16, 24, 8), (4, 520, 5120), (7, 264, 6144), (8, 128, 12288),
                                   (40, 300, 512), (32, 1030, 2048), (17, 264, 2048), (29, 128, 4096),
                                   (24, 72, 200), (32, 12288, 4096), (20, 3000, 4096), (8, 9728, 2560), (6, 200, 2312)])  # fmt: skip
def test_gemm_silu_mul_bf16(ops, M, I, K):
    """Gate and up products with the activation in one kernel (few rows, an input that fits)
    or as product then activation: the same numbers as the two kernels give, which are the plain
    activation of the products rounded to bfloat16."""
    torch.manual_seed(9)
    a, w = torch.randn(M, K, device=DEV).to(BF16), (torch.randn(2 * I, K, device=DEV) / math.sqrt(K)).to(BF16)
    out = torch.empty(M, I, dtype=BF16, device=DEV)
    ops.gemm_silu_mul(a, w, out)
    gate_up = torch.empty(M, 2 * I, dtype=BF16, device=DEV)
    ops.gemm(a, w, gate_up)
    two = torch.empty(M, I, dtype=BF16, device=DEV)
    ops.silu_mul(gate_up, two)
    assert close_bf16(gate_up, pk.gemm(a, w), scale=1.0)
    if M <= 16 or ops._few_rows(M, K, 2 * I) or (M > 32 and not ops._tile_rows(M, K, BF16)):
        assert torch.equal(out, two)  # the same products, whichever kernels made them
        assert close_bf16(out, pk.silu_mul(gate_up))
    else:
        # 17 to 64 wide rows: the gated kernel is this package's, the plain product the library's; their sums
        # differ in the last bit now and then, and the activation carries that on
        assert (out != two).float().mean() < 0.05
        assert torch.allclose(out.float(), pk.silu_mul(pk.gemm(a, w).to(BF16)).float(), atol=2e-2, rtol=2e-2)


def test_every_candidate_of_the_library_gives_the_product(ops):
    """Above the few-rows kernels the product is hipBLASLt's, called directly with one of the
    library's own candidates: each of them is the product, and a shape of a decode bucket settles
    on one of them after trying them in turn."""
    from atomserve_amd.kernels.lib import call, entry

    torch.manual_seed(21)
    workspace = torch.empty(ops.LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=DEV)
    for M, N, K, dtype in ((64, 520, 1024, BF16), (100, 264, 200, F32), (32, 4096, 4096, BF16)):
        a, w = torch.randn(M, K, device=DEV).to(BF16), torch.randn(N, K, device=DEV).to(BF16)
        ref = pk.gemm(a, w)
        count = entry("as_blas_plan")(M, N, K, 0 if dtype == F32 else 1, ops.LIBRARY_WORKSPACE_BYTES)
        assert count >= 1
        for candidate in range(count):
            out = torch.zeros(M, N, dtype=dtype, device=DEV)
            call("as_blas_gemm", a.data_ptr(), w.data_ptr(), out.data_ptr(), 0 if dtype == F32 else 1, M, N, K, candidate,
                 workspace.data_ptr(), ops.LIBRARY_WORKSPACE_BYTES, torch.cuda.current_stream().cuda_stream)  # fmt: skip
            if dtype == BF16:
                assert close_bf16(out, ref, scale=math.sqrt(K)), (M, N, K, candidate)
            else:
                assert torch.allclose(out, ref, atol=math.sqrt(K) * 2.0**-8, rtol=2.0**-7), (M, N, K, candidate)
        with pytest.raises(ops.KernelError):
            call("as_blas_gemm", a.data_ptr(), w.data_ptr(), out.data_ptr(), 1, M, N, K, count, workspace.data_ptr(),
                 ops.LIBRARY_WORKSPACE_BYTES, torch.cuda.current_stream().cuda_stream)  # fmt: skip
    # 64 rows is a decode bucket: the first calls try the candidates, then one stays
    M, N, K = 64, 528, 8192
    a, w = torch.randn(M, K, device=DEV).to(BF16), torch.randn(N, K, device=DEV).to(BF16)
    ref = pk.gemm(a, w)
    out = torch.empty(M, N, dtype=BF16, device=DEV)
    for _ in range(ops.LIBRARY_TRIALS_EACH * 16 + 2):
        out.zero_()
        ops.gemm(a, w, out)
        assert close_bf16(out, ref, scale=math.sqrt(K))
    assert (M, N, K, BF16) in ops.SHARED.chosen()
    ops.SHARED.settle()  # and whatever other tests left half tried
    assert not ops.SHARED.trials_pending()
    # choices are a model's own: another object starts with none, and fixed takes the first candidate
    mine = ops.ProductChoices(fixed=True)
    out.zero_()
    ops.gemm(a, w, out, mine)
    assert close_bf16(out, ref, scale=math.sqrt(K)) and mine.chosen() == {(M, N, K, BF16): 0}


def test_a_product_of_any_row_count_takes_what_the_tuned_count_above_it_chose(ops):
    """Prompts come in every length: a product whose row count is not tuned itself runs the kernel that
    the nearest tuned row count above it settled on (by the library's own number of that kernel), and
    gives the product; while that one is undecided, and with fixed choices, the first candidate."""
    from atomserve_amd.kernels.lib import entry

    torch.manual_seed(31)
    N, K, tuned, M = 1024, 2048, 192, 100
    w = torch.randn(N, K, device=DEV).to(BF16)
    a = torch.randn(M, K, device=DEV).to(BF16)
    out = torch.empty(M, N, dtype=BF16, device=DEV)
    number = lambda rows, place: entry("as_blas_candidate_index")(rows, N, K, 1, ops.LIBRARY_WORKSPACE_BYTES, place)
    choices = ops.ProductChoices()
    choices.tune_rows(tuned)
    ops.gemm(a, w, out, choices)  # nothing settled above 100 rows: the first candidate, and no decision
    assert close_bf16(out, pk.gemm(a, w), scale=math.sqrt(K)) and (M, N, K, BF16) not in choices.chosen()
    big = torch.randn(tuned, K, device=DEV).to(BF16)
    big_out = torch.empty(tuned, N, dtype=BF16, device=DEV)
    while (tuned, N, K, BF16) not in choices.chosen():
        ops.gemm(big, w, big_out, choices)
    chosen = choices.chosen()[(tuned, N, K, BF16)]
    out.fill_(float("nan"))
    ops.gemm(a, w, out, choices)
    assert close_bf16(out, pk.gemm(a, w), scale=math.sqrt(K))
    mine = choices.chosen()[(M, N, K, BF16)]
    assert number(M, mine) == number(tuned, chosen) or (mine == 0 and entry("as_blas_adopt")(M, N, K, 1, ops.LIBRARY_WORKSPACE_BYTES, number(tuned, chosen)) < 0)
    # a kernel that this shape's own list does not hold is added to it, once
    count = entry("as_blas_plan")(M + 1, N, K, 1, ops.LIBRARY_WORKSPACE_BYTES)
    for place in range(entry("as_blas_plan")(tuned, N, K, 1, ops.LIBRARY_WORKSPACE_BYTES)):
        at = entry("as_blas_adopt")(M + 1, N, K, 1, ops.LIBRARY_WORKSPACE_BYTES, number(tuned, place))
        assert at < 0 or number(M + 1, at) == number(tuned, place)
        assert at == entry("as_blas_adopt")(M + 1, N, K, 1, ops.LIBRARY_WORKSPACE_BYTES, number(tuned, place))
    grown = entry("as_blas_plan")(M + 1, N, K, 1, ops.LIBRARY_WORKSPACE_BYTES)
    assert grown >= count
    a1 = torch.randn(M + 1, K, device=DEV).to(BF16)
    for place in range(count, grown):  # the adopted ones give the product too
        o1 = torch.zeros(M + 1, N, dtype=BF16, device=DEV)
        ops._library_call(a1, w, o1, M + 1, N, K, place)
        assert close_bf16(o1, pk.gemm(a1, w), scale=math.sqrt(K)), place
    assert entry("as_blas_adopt")(M + 1, N, K, 1, ops.LIBRARY_WORKSPACE_BYTES, -1) < 0
    assert ops.prepare_library_adoption()  # the look-up by number that a warm-up makes ahead of serving
    assert (tuned, N, K, BF16) not in ops.SHARED.chosen() and tuned not in ops.SHARED.tuned_rows  # nobody else's business


@pytest.mark.parametrize("M,N,K", [(48, 544, 1024), (9, 544, 1024), (12, 6144, 4096), (16, 1024, 2560), (128, 48, 256)])
def test_the_tile_product_is_a_candidate_beside_the_librarys(ops, M, N, K):
    """For 9 to 128 rows and weights with a copy in wave order, a trial also times this package's plain tile
    product (tiles of 2 and 4 strips); chosen, it gives the product, and weights without a copy fall back
    to the library's first candidate under the same choice."""
    torch.manual_seed(5)
    a = torch.randn(M, K, device=DEV).to(BF16)
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).to(BF16)
    bare = w.clone()
    assert ops._own_candidates(M, N, K, BF16, w) == [] and ops._own_candidates(M, N, K, BF16, ops.Streamed(w, copy=False)) == []
    w = ops.Streamed(w)  # with its copy in wave order
    own = ops._own_candidates(M, N, K, BF16, w)
    assert own == [ops.OWN_CANDIDATE + 2, ops.OWN_CANDIDATE + 4]
    assert ops._own_candidates(M, N + 8, K, BF16, None) == [] and ops._own_candidates(8, N, K, BF16, None) == []
    assert ops._own_candidates(M, N, K + 64, BF16, None) == [] and ops._own_candidates(129, N, K, BF16, None) == []
    ref = pk.gemm(a, bare)
    key = (M, N, K, BF16)
    for candidate in own:
        choices = ops.ProductChoices()
        choices.tune_rows(M)
        out = torch.full((M, N), float("nan"), dtype=BF16, device=DEV)
        ops._library_call(a, w, out, M, N, K, candidate)
        assert close_bf16(out, ref, scale=1.0)
        choices.gemm(a, w, out, M, N, K)  # makes the library's plan and workspace for this shape, and starts a trial
        assert choices.trials[key]["ids"][-2:] == own  # this package's products are tried beside the library's
        choices.trials.clear()
        choices.choice[key] = candidate
        for weights in (w, bare):
            out.fill_(float("nan"))
            choices.gemm(a, weights, out, M, N, K)
            assert close_bf16(out, ref, scale=1.0)


def test_library_candidates_replay_from_a_graph(ops):
    """Each candidate captured once and replayed with other inputs and a workspace full of noise,
    with eager work and synchronisations between the replays: every replay gives what the eager
    call gives (a candidate that clears its workspace through a captured memset would not)."""
    from atomserve_amd.kernels.lib import call, entry

    size = ops.LIBRARY_WORKSPACE_BYTES
    workspace = torch.empty(size, dtype=torch.uint8, device=DEV)
    for M, N, K in ((64, 4096, 4096), (32, 4096, 12288), (64, 1024, 3072)):
        torch.manual_seed(M + K)
        w = (torch.randn(N, K, device=DEV) * 0.02).to(BF16)
        a = torch.randn(M, K, device=DEV).to(BF16)
        out = torch.empty(M, N, dtype=BF16, device=DEV)
        for candidate in range(entry("as_blas_plan")(M, N, K, 1, size)):
            def run():
                call("as_blas_gemm", a.data_ptr(), w.data_ptr(), out.data_ptr(), 1, M, N, K, candidate,
                     workspace.data_ptr(), size, torch.cuda.current_stream().cuda_stream)  # fmt: skip

            run()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                run()
            for _ in range(3):
                a.copy_(torch.randn(M, K, device=DEV).to(BF16))
                workspace[: 1 << 20].random_(0, 255)
                out.zero_()
                graph.replay()
                torch.cuda.synchronize()
                replayed = out.clone()
                workspace[: 1 << 20].random_(0, 255)
                out.zero_()
                run()
                torch.cuda.synchronize()
                assert torch.equal(replayed, out), (M, N, K, candidate)


def test_gemm_silu_mul_fp32(ops):
    torch.manual_seed(10)
    a, w = torch.randn(5, 72, device=DEV), torch.randn(2 * 50, 72, device=DEV) / 8
    out = torch.empty(5, 50, device=DEV)
    ops.gemm_silu_mul(a, w, out)
    assert torch.allclose(out, pk.silu_mul(pk.gemm(a, w)), atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("M,N,K", [(1, 96, 64), (8, 1000, 96), (5, 1032, 4096), (16, 4096, 4096), (3, 40, 200),
                                   (16, 24, 8), (8, 520, 12288), (13, 304, 6152), (4, 4096, 6144), (32, 1024, 4096),
                                   (17, 1032, 12288), (27, 520, 200), (32, 2048, 4104), (20, 40, 2048), (8, 2560, 2560),
                                   (12, 2560, 9728)])  # fmt: skip
def test_gemm_link_bf16(ops, M, N, K):
    """The product that adds into the fp32 stream and prepares the next norm: the stream receives
    exactly the product kernel's bf16 output; beside it x * gain rounded to bf16 and the sums of
    x^2 per 16 columns."""
    assert ops.gemm_link_supported(M, N, K, BF16)
    torch.manual_seed(12)
    a, w = torch.randn(M, K, device=DEV).to(BF16), torch.randn(N, K, device=DEV).to(BF16)
    gain = torch.randn(N, device=DEV) * 0.3 + 1
    x0 = torch.randn(M, N, device=DEV) * 50
    x = x0.clone()
    scaled = torch.zeros(M, N, dtype=BF16, device=DEV)
    strips = -(-N // 16)
    ssq = torch.zeros(M, strips, device=DEV)
    ops.gemm_link(a, w, x, gain, scaled, ssq)
    if M <= 16 or (K <= ops.SKINNY_TWO_MAX_K and ops._few_rows(M, K, N)):  # the plain product sums in the same order
        y = torch.empty(M, N, dtype=BF16, device=DEV)
        ops.gemm(a, w, y)
        assert torch.equal(x, x0 + y.float())
    else:  # what the stream received is the product rounded to bf16 (the fp32 sum's own rounding is far below)
        assert close_bf16(x - x0, pk.gemm(a, w), scale=math.sqrt(K))
    assert torch.equal(scaled, (x * gain).to(BF16))
    padded = torch.zeros(M, strips * 16, device=DEV)
    padded[:, :N] = x
    assert torch.allclose(ssq, (padded.double() ** 2).view(M, strips, 16).sum(-1).float(), rtol=1e-5)


@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("M,N,K", [(1, 96, 64), (8, 1000, 96), (5, 1030, 4096), (16, 6144, 4096), (9, 700, 2048),
                                   (3, 40, 200), (16, 24, 8), (7, 264, 3072), (2, 130, 5120), (32, 6144, 1024),
                                   (17, 1030, 2048), (26, 40, 200), (31, 264, 2048), (6, 6148, 4096), (20, 6144, 2048),
                                   (8, 6144, 2560), (3, 100, 2400)])  # fmt: skip
def test_gemm_scaled_bf16(ops, M, N, K, gated):
    """The product that finishes a pending norm: x * gain arrives rounded to bf16, 1 / rms comes
    from the sums of squares and multiplies the fp32 sums.  That input times the plain 1 / rms is
    the plain norm up to its rounding; the plain product of it (and the activation) is met within
    the product's own tolerance.  One row is a thousand times larger than the others, so a factor
    taken from the wrong row shows."""
    torch.manual_seed(11)
    x = torch.randn(M, K, device=DEV) * 3
    x[M // 2] *= 1000.0
    gain = torch.randn(K, device=DEV) * 0.3 + 1
    eps = 1e-5
    w = (torch.randn((2 if gated else 1) * N, K, device=DEV) / (math.sqrt(K) if gated else 1.0)).to(BF16)
    strips = -(-K // 16)
    padded = torch.zeros(M, strips * 16, device=DEV)
    padded[:, :K] = x
    ssq = (padded**2).view(M, strips, 16).sum(-1).contiguous()
    out = torch.empty(M, N, dtype=BF16, device=DEV)
    # the plain norm and product, on the input as the kernel gets it: x * gain rounded to bf16
    scaled = (x * gain).to(BF16)
    normed, _ = pk.rmsnorm(x, gain, eps)
    inv_rms = 1.0 / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + eps)
    assert close_bf16(scaled.double() * inv_rms, normed)
    ref = ((scaled.double() @ w.double().T) * inv_rms).float()
    ops.gemm_scaled(scaled, ssq, eps, w, out, gated=gated)
    if not gated:
        assert close_bf16(out, ref, scale=math.sqrt(K))
        return
    # each of the two products within the product's tolerance (its sums have a deviation of one
    # here), carried through silu(g) * u: |d silu| <= 1.1 |dg|
    g, u = ref.double().chunk(2, dim=-1)
    err_g, err_u = g.abs() * 2.0**-7 + 2.0**-8, u.abs() * 2.0**-7 + 2.0**-8
    silu = g / (1 + torch.exp(-g))
    want = silu * u
    bound = 1.1 * u.abs() * err_g + silu.abs() * err_u + 1.1 * err_g * err_u + want.abs() * 2.0**-8
    assert bool(((out.double() - want).abs() <= bound).all())


@pytest.mark.parametrize("M,N,K", [(1, 96, 512), (8, 1024, 4096), (5, 4096, 1024), (16, 608, 2048), (3, 48, 6144), (8, 4096, 12288),
                                   (13, 304, 6400), (16, 64, 8192), (32, 256, 1024), (20, 144, 2048), (17, 1024, 12288), (8, 32, 3072),
                                   (7, 80, 5120), (8, 96, 64), (4, 64, 576), (8, 40, 512), (8, 48, 520), (8, 512, 2560),
                                   (16, 9728, 2560), (8, 2560, 9728)])  # fmt: skip
def test_weights_in_wave_order_give_the_same_products(ops, M, N, K):
    """The copy of a weight matrix in the order in which a wave reads it holds the same values at the places
    the kernels' indexing says, and every few-rows product that finds such a copy on its weights gives bit for
    bit what it gives from rows (the same values reach the same lanes).  Sizes of both few-rows kernels,
    whole and partial workgroup rounds, one and two row tiles; sizes that take no copy go on as before."""
    torch.manual_seed(M * 7 + N)
    values = (torch.randn(2 * N, K, device=DEV) / math.sqrt(K)).to(BF16)
    w = ops.Streamed(values)
    copy = w.wave
    if (2 * N) % 16 or K % 64:
        assert copy is None and w.wave_bytes == 0 and not ops.Streamed.possible(values)
        return
    want = values.view(2 * N // 16, 16, K // 64, 4, 2, 8).permute(0, 2, 4, 3, 1, 5).contiguous().view(2 * N, K)  # strip, step, half, lane / 16, lane % 16
    assert torch.equal(copy, want) and w.rows is values and w.wave_bytes == values.numel() * 2
    assert ops.Streamed(values, copy=False).wave is None  # the owner asked for none
    plain = values.clone()  # the same values without a copy
    a = torch.randn(M, K, device=DEV).to(BF16)

    def both(run, *outs):
        """run(weights, *outputs) with the copy and without: equal outputs."""
        got = [o.clone() for o in outs]
        run(w, *got)
        ref = [o.clone() for o in outs]
        run(plain, *ref)
        for g, r in zip(got, ref):
            assert torch.equal(g, r)
        return got

    for dtype in (BF16, F32):
        if ops._few_rows(M, K, 2 * N, w=w):
            both(lambda wt, out: ops.gemm(a, wt, out), torch.empty(M, 2 * N, dtype=dtype, device=DEV))
        elif ops._few_rows(M, K, 2 * N) and dtype == BF16:
            # 17 to 32 rows: from rows the persistent kernel with two row tiles, with the copy the tile products or the library
            with_copy, from_rows = torch.empty(M, 2 * N, dtype=BF16, device=DEV), torch.empty(M, 2 * N, dtype=BF16, device=DEV)
            ops.gemm(a, w, with_copy)
            ops.gemm(a, plain, from_rows)
            assert close_bf16(with_copy, from_rows.double(), scale=1.0)
    if ops._few_rows(M, K, N, ops.GATED_MAX_K, w=w):
        both(lambda wt, out: ops.gemm_silu_mul(a, wt, out), torch.empty(M, N, dtype=BF16, device=DEV))
    elif ops._few_rows(M, K, N, ops.GATED_MAX_K) or ops._gated_two_tiles(M, K, plain):
        # 17 to 32 rows: from rows the persistent kernel with two row tiles, with the copy the tile product
        assert not ops._gated_two_tiles(M, K, w)
        with_copy, from_rows = torch.empty(M, N, dtype=BF16, device=DEV), torch.empty(M, N, dtype=BF16, device=DEV)
        ops.gemm_silu_mul(a, w, with_copy)
        ops.gemm_silu_mul(a, plain, from_rows)
        assert torch.allclose(with_copy.float(), from_rows.float(), atol=2e-2, rtol=2e-2)
    if ops.gemm_link_supported(M, 2 * N, K, BF16):
        gain = torch.randn(2 * N, device=DEV) * 0.3 + 1
        x0 = torch.randn(M, 2 * N, device=DEV)
        both(lambda wt, x, scaled, ssq: ops.gemm_link(a, wt, x, gain, scaled, ssq), x0,
             torch.zeros(M, 2 * N, dtype=BF16, device=DEV), torch.zeros(M, 2 * N // 16, device=DEV))
    if ops.gemm_link_supported(M, K, 8, BF16):
        ssq = (a.float() ** 2).view(M, K // 16, 16).sum(-1).contiguous()
        for gated in (False, True):
            both(lambda wt, out: ops.gemm_scaled(a, ssq, 1e-5, wt, out, gated=gated),
                 torch.empty(M, N if gated else 2 * N, dtype=BF16, device=DEV))
    # a matrix changed in place takes its copy anew when its owner says so, and the products follow
    values.mul_(2)
    assert torch.equal(w.wave, want)  # stale until then
    assert torch.equal(w.refresh(), (want.float() * 2).to(BF16)) and w.wave is copy
    if ops._few_rows(M, K, 2 * N, w=w):
        got, ref = torch.empty(M, 2 * N, dtype=BF16, device=DEV), torch.empty(M, 2 * N, dtype=BF16, device=DEV)
        ops.gemm(a, w, got)
        ops.gemm(a, values.clone(), ref)
        assert torch.equal(got, ref)


def test_gemm_link_refuses_what_it_cannot_do(ops):
    assert not ops.gemm_link_supported(33, 1024, 1024, BF16)
    assert not ops.gemm_link_supported(32, 4096, 4096, BF16)  # two row tiles of such rows in 256 workgroups: more bytes than the weights
    assert ops.gemm_link_supported(32, 1024, 3072, BF16)
    assert not ops.gemm_link_supported(8, 4100, 4096, BF16)
    assert not ops.gemm_link_supported(8, 8192, 4096, BF16)  # the next product could not keep such rows in registers
    assert not ops.gemm_link_supported(8, 4096, 4096, F32)
    a, w = torch.zeros(8, 64, dtype=BF16, device=DEV), torch.zeros(8192, 64, dtype=BF16, device=DEV)
    with pytest.raises(ops.KernelError):
        ops.gemm_link(a, w, torch.zeros(8, 8192, device=DEV), torch.ones(8192, device=DEV),
                      torch.zeros(8, 8192, dtype=BF16, device=DEV), torch.zeros(8, 512, device=DEV))


def paged_case(dtype, H, KV, D, bs, lens, seed=0, k_scale=4.0):
    """Random pools and scattered block tables for contexts of the given lengths; the query of
    request i sits at position lens[i] - 1."""
    g = torch.Generator().manual_seed(seed)
    pages = sum(-(-n // bs) for n in lens) + 8
    k_pages = (torch.randn(pages, KV, bs, D, generator=g) * k_scale).to(dtype).to(DEV)
    v_pages = torch.randn(pages, KV, D, bs, generator=g).to(dtype).to(DEV)  # values transposed within a page
    perm = torch.randperm(pages, generator=g).tolist()
    tables, at = [], 0
    for n in lens:
        nb = -(-n // bs)
        tables.append(perm[at : at + nb])
        at += nb
    width = max(map(len, tables))
    padded = i32([t + [0] * (width - len(t)) for t in tables])
    q = torch.randn(len(lens), H, D, generator=g).to(dtype).to(DEV)
    positions = i32([n - 1 for n in lens])
    return q, k_pages, v_pages, padded, positions


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("H,KV,D,bs", [(16, 8, 128, 16), (32, 8, 128, 16), (8, 8, 128, 16), (6, 2, 32, 8),
                                       (4, 2, 16, 16), (5, 1, 48, 4), (16, 1, 64, 32), (64, 8, 128, 16),
                                       (16, 1, 256, 16), (32, 2, 256, 16)])  # fmt: skip
def test_attention_single_query(ops, dtype, H, KV, D, bs):
    """Contexts of one key, part of a page, exactly one partition and several partitions, on
    scattered pages (lengths from reference tests/test_kernels.py:98-125)."""
    if dtype == BF16 and D % 8:
        pytest.skip("bf16 heads come in steps of 8")
    lens = [1, 37, 512, 513, 1500]
    q, k_pages, v_pages, tables, positions = paged_case(dtype, H, KV, D, bs, lens, k_scale=4.0 / math.sqrt(D / 16))
    rows = i32(list(range(len(lens))))
    items = i32(list(range(len(lens))))
    out = torch.zeros(len(lens), H, D, dtype=dtype, device=DEV)
    scale = D**-0.5
    ref = pk.paged_attention(q, k_pages, v_pages, items, positions, rows, tables, scale)
    for part_size, generic in ((None, False), (256, False), (64, False), (None, True), (64, True)):
        out.zero_()
        ops.attn_single_query(q, k_pages, v_pages, items, positions, rows, tables, out, scale, 0, max(lens), part_size,
                              force_generic=generic)  # fmt: skip
        if dtype == F32:
            assert torch.allclose(out, ref, atol=1e-5), f"partitions of {part_size}: {(out - ref).abs().max()}"
        else:
            assert torch.allclose(out.float(), ref, atol=2e-2, rtol=2e-2), f"{part_size, generic}: {(out.float() - ref).abs().max()}"


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_attention_finds_one_far_key_among_many(ops, dtype):
    """One key far back matches the query strongly; the result must be (almost) that key's value,
    wherever in the context, the pages and the partitions it lies."""
    H, KV, D, bs, n = 8, 2, 64, 16, 1500
    for far in (0, 15, 16, 255, 256, 700, 1498, 1499):
        q, k_pages, v_pages, tables, positions = paged_case(dtype, H, KV, D, bs, [n], seed=far, k_scale=0.05)
        page, off = int(tables[0, far // bs]), far % bs
        G = H // KV
        for kvh in range(KV):  # the first query head of each group gets its match
            k_pages[page, kvh, off] = (q[0, kvh * G].float() * 4.0).to(dtype)
        for generic in (False, True):
            out = torch.zeros(1, H, D, dtype=dtype, device=DEV)
            ops.attn_single_query(q, k_pages, v_pages, i32([0]), positions, i32([0]), tables, out, 1.0, 0, n,
                                  force_generic=generic)  # fmt: skip
            for kvh in range(KV):
                want = v_pages[page, kvh, :, off].float()
                assert torch.allclose(out[0, kvh * G].float(), want, atol=2e-2), (far, kvh, generic)


@pytest.mark.parametrize("window", [1, 5, 16, 17, 300])
@pytest.mark.parametrize("dtype,bs", [(F32, 8), (BF16, 16)])
def test_attention_window_edge(ops, window, dtype, bs):
    H, KV, D = 4, 2, 32
    lens = [1, 9, 100, 513]
    q, k_pages, v_pages, tables, positions = paged_case(dtype, H, KV, D, bs, lens)
    items = rows = i32(list(range(4)))
    out = torch.zeros(4, H, D, dtype=dtype, device=DEV)
    ops.attn_single_query(q, k_pages, v_pages, items, positions, rows, tables, out, D**-0.5, window, max(lens), 64)
    ref = pk.paged_attention(q, k_pages, v_pages, items, positions, rows, tables, D**-0.5, window)
    assert torch.allclose(out.float(), ref, atol=1e-5 if dtype == F32 else 2e-2)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_attention_of_a_decode_step_needs_no_maps(ops, dtype):
    """Every token is a row of its own: without the token list and the token-to-row map the
    kernels do exactly what they do with the identity maps."""
    H, KV, D, bs = 8, 2, 64, 16
    lens = [1, 37, 300, 513]
    q, k_pages, v_pages, tables, positions = paged_case(dtype, H, KV, D, bs, lens, seed=7)
    ident = i32(list(range(4)))
    a = torch.zeros(4, H, D, dtype=dtype, device=DEV)
    b = torch.zeros_like(a)
    for part in (None, 64):
        ops.attn_single_query(q, k_pages, v_pages, ident, positions, ident, tables, a, D**-0.5, 0, max(lens), part)
        ops.attn_single_query(q, k_pages, v_pages, None, positions, None, tables, b, D**-0.5, 0, max(lens), part)
        assert torch.equal(a, b)
    with pytest.raises(ops.KernelError):
        ops.attn_single_query(q, k_pages, v_pages, None, positions, None, tables[:3], b, D**-0.5, 0, max(lens))


@pytest.mark.parametrize("N,KV", [(40, 8), (100, 8), (70, 3), (300, 2), (5, 8)])
def test_whole_contexts_in_a_given_order(ops, N, KV):
    """Single queries over whole contexts (no partitions), more workgroups than one, two and three rounds
    of one per compute unit, taken in the order of a permutation (longest first, as a decode step packs
    them, and a random one): every token is attended exactly once, by both kernels' entry points."""
    H, D, bs = 2 * KV, 64, 16
    torch.manual_seed(N)
    lens = torch.randint(1, 200, (N,)).tolist()
    q, k_pages, v_pages, tables, positions = paged_case(BF16, H, KV, D, bs, lens, seed=N, k_scale=3.0 / math.sqrt(D / 16))
    rows = i32(list(range(N)))
    scale = D**-0.5
    ref = pk.paged_attention(q, k_pages, v_pages, rows, positions, rows, tables, scale, 0)
    whole = -(-max(lens) // 32) * 32
    longest_first = torch.argsort(positions, descending=True, stable=True).to(torch.int32)
    shuffled = torch.randperm(N).to(torch.int32).to(DEV)
    for order in (None, longest_first, shuffled):
        out = torch.full((N, H, D), float("nan"), dtype=BF16, device=DEV)
        ops.attn_single_query(q, k_pages, v_pages, order, positions, None, tables, out, scale, 0, max(lens), whole)
        assert torch.allclose(out.float(), ref, atol=2e-2, rtol=2e-2)
    # the kernel fed with fresh projections, queries only (the pages hold the keys already)
    g = torch.Generator().manual_seed(N + 1)
    qkv = (torch.randn(N, H + 2 * KV, D, generator=g) * 2).to(BF16).to(DEV)
    qw, kw = (torch.randn(D, generator=g) + 1).to(BF16).to(DEV), (torch.randn(D, generator=g) + 1).to(BF16).to(DEV)
    inv = (1.0 / (1e4 ** (torch.arange(0, D, 2, dtype=torch.float64) / D))).to(DEV)
    cs = torch.empty(N, D // 2, 2, device=DEV)
    ops.rope_table(positions, inv, cs)
    outs = []
    for order in (None, longest_first, shuffled):
        out = torch.full((N, H, D), float("nan"), dtype=BF16, device=DEV)
        ops.attn_decode_fresh(qkv, qw, kw, cs, None, 1e-6, False, k_pages, v_pages, positions, tables, out, H, scale, 0,
                              max(lens), whole, order=order)
        outs.append(out)
    assert not torch.isnan(outs[0].float()).any()
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])


@pytest.mark.parametrize("H,KV,D,bs,gain,window", [
    (32, 8, 128, 16, BF16, 0), (6, 2, 64, 32, F32, 0), (14, 2, 192, 16, BF16, 40), (5, 5, 256, 16, BF16, 0),
    (16, 1, 128, 48, F32, 0), (8, 2, 128, 16, BF16, 1),
])  # fmt: skip
@pytest.mark.parametrize("part", [None, 32, 128])
def test_decode_step_from_fresh_projections(ops, H, KV, D, bs, gain, window, part):
    """Norm, rotation, cache store and attention of a decode step in one kernel: against the plain
    functions, and against the two kernels it stands for.  Contexts end at the first and the last
    slot of a page, at the edges of the partitions and of a wave's 32 keys; one row keeps its token
    out of the pages (slot -1) and still attends it; with `store_kv` off nothing is written and the
    key that the pages hold is attended."""
    lens = [1, 16, 17, 32, 33, 128, 129, 300, 512, 513, 1000]
    _, k_pages, v_pages, tables, positions = paged_case(BF16, H, KV, D, bs, lens, seed=5, k_scale=3.0 / math.sqrt(D / 16))
    T = len(lens)
    g = torch.Generator().manual_seed(9)
    qkv = (torch.randn(T, H + 2 * KV, D, generator=g) * 2).to(BF16).to(DEV)
    qw, kw = (torch.randn(D, generator=g) + 1).to(gain).to(DEV), (torch.randn(D, generator=g) + 1).to(gain).to(DEV)
    inv = (1.0 / (1e4 ** (torch.arange(0, D, 2, dtype=torch.float64) / D))).to(DEV)
    cs = torch.empty(T, D // 2, 2, device=DEV)
    ops.rope_table(positions, inv, cs)
    slot_list = [tables[i, (n - 1) // bs].item() * bs + (n - 1) % bs for i, n in enumerate(lens)]
    slot_list[3] = -1  # this row's token stays out of the pages
    slots = i32(slot_list)
    scale = D**-0.5
    rows = i32(list(range(T)))
    # plain: the new keys and values go to the pages, then every query attends its context
    rq, rk, rv = pk.qk_norm_rope(qkv, qw, kw, cs, H, KV, 1e-6)
    ref_k, ref_v = k_pages.float(), v_pages.float()
    pk.store_pages(ref_k, ref_v, rk, rv, i32([tables[i, (n - 1) // bs].item() * bs + (n - 1) % bs for i, n in enumerate(lens)]))
    ref = pk.paged_attention(rq.to(BF16), ref_k.to(BF16), ref_v.to(BF16), rows, positions, rows, tables, scale, window)
    # the two kernels
    k2, v2 = k_pages.clone(), v_pages.clone()
    q2, out2 = torch.empty(T, H, D, dtype=BF16, device=DEV), torch.zeros(T, H, D, dtype=BF16, device=DEV)
    ops.qk_norm_rope_store(qkv, qw, kw, cs, slots, q2, k2, v2, H, KV, 1e-6)
    ops.attn_single_query(q2, k2, v2, None, positions, None, tables, out2, scale, window, max(lens), part)
    # the one kernel
    k1, v1 = k_pages.clone(), v_pages.clone()
    out1 = torch.zeros(T, H, D, dtype=BF16, device=DEV)
    ops.attn_decode_fresh(qkv, qw, kw, cs, slots, 1e-6, True, k1, v1, positions, tables, out1, H, scale, window, max(lens), part)
    torch.cuda.synchronize()
    assert torch.equal(v1, v2)
    assert close_bf16(k1, k2.float()) and (k1 != k2).float().mean() < 0.02  # the squares are summed in another order
    written = torch.zeros(k_pages.shape[0] * bs, dtype=torch.bool, device=DEV)
    written[slots[slots >= 0].long()] = True
    untouched = ~written.view(-1, bs)  # [page, offset]: nothing but the slots was written
    assert torch.equal(k1.permute(0, 2, 1, 3)[untouched], k_pages.permute(0, 2, 1, 3)[untouched])
    assert torch.equal(v1.permute(0, 3, 1, 2)[untouched], v_pages.permute(0, 3, 1, 2)[untouched])
    assert torch.allclose(out1.float(), ref, atol=2e-2, rtol=2e-2)
    keep = [i for i in range(T) if i != 3]  # the two kernels cannot attend a token that they keep out of the pages
    assert torch.allclose(out1[keep].float(), out2[keep].float(), atol=2e-2, rtol=2e-2)
    # queries only: the pages as the plain store left them are read, nothing is written
    k3, v3 = ref_k.to(BF16), ref_v.to(BF16)
    before_k, before_v = k3.clone(), v3.clone()
    out3 = torch.zeros(T, H, D, dtype=BF16, device=DEV)
    ops.attn_decode_fresh(qkv, qw, kw, cs, None, 1e-6, False, k3, v3, positions, tables, out3, H, scale, window, max(lens), part)
    torch.cuda.synchronize()
    assert torch.equal(k3, before_k) and torch.equal(v3, before_v)
    assert torch.allclose(out3.float(), ref, atol=2e-2, rtol=2e-2)
    # heads without a norm or a whole rotation are left to the two kernels
    for weights, angles in ((None, cs), (qw, None), (qw, cs[:, : D // 4].contiguous())):
        with pytest.raises(ops.KernelError, match="fresh projections"):
            ops.attn_decode_fresh(qkv, weights, weights, angles, slots, 1e-6, True, k3, v3, positions, tables, out3, H,
                                  scale, window, max(lens), part)  # fmt: skip


def test_attention_of_a_batch_that_fills_the_gpu(ops):
    """64 requests of 8 kv heads are 512 workgroups already: the contexts are not partitioned (no
    merge), each workgroup walks its whole context, of very different lengths."""
    H, KV, D, bs = 16, 8, 64, 16
    lens = [1 + (37 * i * i) % 1400 for i in range(64)]
    assert 64 * KV >= ops.attn_fill_groups()
    q, k_pages, v_pages, tables, positions = paged_case(BF16, H, KV, D, bs, lens, seed=5, k_scale=1.0)
    out = torch.zeros(64, H, D, dtype=BF16, device=DEV)
    ops.attn_single_query(q, k_pages, v_pages, None, positions, None, tables, out, D**-0.5, 0, max(lens))
    rows = i32(list(range(64)))
    ref = pk.paged_attention(q, k_pages, v_pages, rows, positions, rows, tables, D**-0.5)
    assert torch.allclose(out.float(), ref, atol=2e-2, rtol=2e-2)


def test_attention_serves_only_the_listed_tokens(ops):
    """Items select tokens; several tokens of one request share a table and see keys up to
    their own position only."""
    H, KV, D, bs = 4, 2, 32, 8
    q, k_pages, v_pages, tables, _ = paged_case(F32, H, KV, D, bs, [40])
    q = torch.randn(6, H, D, device=DEV)
    positions, rows = i32([3, 4, 5, 37, 38, 39]), i32([0] * 6)
    items = i32([1, 4, 5])
    out = torch.full((6, H, D), 9.0, device=DEV)
    ops.attn_single_query(q, k_pages, v_pages, items, positions, rows, tables, out, D**-0.5, 0, 40)
    ref = pk.paged_attention(q, k_pages, v_pages, items, positions, rows, tables, D**-0.5)
    assert torch.allclose(out[[1, 4, 5]], ref[[1, 4, 5]], atol=1e-5)
    assert bool((out[[0, 2, 3]] == 9.0).all())


@pytest.mark.parametrize("H,KV,D,bs,window", [(32, 8, 128, 16, 0), (6, 2, 32, 16, 0), (8, 8, 64, 32, 0), (4, 1, 96, 16, 0),
                                               (16, 2, 128, 16, 0), (4, 2, 64, 16, 40), (4, 2, 64, 16, 1), (4, 2, 256, 16, 0),
                                               (2, 1, 224, 32, 0), (10, 2, 160, 16, 70)])  # fmt: skip
def test_attention_prefill(ops, H, KV, D, bs, window):
    """Prompt portions that start at position 0 and after a cached prefix, of lengths around
    the tile sizes (16, 32, 64), each query seeing keys up to its own position."""
    torch.manual_seed(12)
    rows = [(0, 70), (37, 9), (100, 64), (5, 130), (300, 33), (0, 16), (511, 17)]  # (start, new tokens)
    lens = [a + n for a, n in rows]
    _, k_pages, v_pages, tables, _ = paged_case(BF16, H, KV, D, bs, lens, seed=3, k_scale=2.0 / math.sqrt(D / 16))
    T = sum(n for _, n in rows)
    q = torch.randn(T, H, D, device=DEV).to(BF16)
    positions, tok_row, tiles, flat = [], [], [], 0
    for r, (start, n) in enumerate(rows):
        positions += list(range(start, start + n))
        tok_row += [r] * n
        for q0 in range(0, n, 64):
            tiles.append([flat + q0, min(64, n - q0), r, start + q0])
        flat += n
    ref = pk.paged_attention(q, k_pages, v_pages, i32(list(range(T))), i32(positions), i32(tok_row), tables, D**-0.5, window)
    for query_tiles, cut in [(None, None), (1, 1), (2, 1), (1, 2), (2, 3), (2, 4)]:  # as the sizes choose; a wave owning 16 queries; 32; long items cut into pieces
        out = torch.zeros(T, H, D, dtype=BF16, device=DEV)
        with prefill_cut(ops, cut):
            ops.attn_prefill(q, k_pages, v_pages, i32(tiles), tables, out, D**-0.5, window, max(lens), query_tiles=query_tiles)
        assert torch.allclose(out.float(), ref, atol=2e-2, rtol=2e-2), (query_tiles, cut, (out.float() - ref).abs().max())


def test_attention_prefill_of_a_long_prompt_in_one_step(ops):
    """4,500 tokens at once after a prefix of 700: many more work items than the GPU holds at a
    time, in the order the engine gives them (most keys first), hundreds of rounds per item."""
    H, KV, D, bs, start, n = 8, 2, 128, 16, 700, 4500
    torch.manual_seed(15)
    _, k_pages, v_pages, tables, _ = paged_case(BF16, H, KV, D, bs, [start + n], seed=9, k_scale=2.0 / math.sqrt(D / 16))
    q = torch.randn(n, H, D, device=DEV).to(BF16)
    tiles = sorted(([q0, min(64, n - q0), 0, start + q0] for q0 in range(0, n, 64)), key=lambda t: -(t[3] + t[1]))
    check = list(range(0, n, 97)) + [n - 1]
    ref = pk.paged_attention(q, k_pages, v_pages, i32(check), i32(list(range(start, start + n))), i32([0] * n), tables, D**-0.5)
    for query_tiles, cut in ((2, 1), (1, 1), (2, 2), (1, 5)):
        out = torch.zeros(n, H, D, dtype=BF16, device=DEV)
        with prefill_cut(ops, cut):
            ops.attn_prefill(q, k_pages, v_pages, i32(tiles), tables, out, D**-0.5, 0, start + n, query_tiles=query_tiles)
        assert torch.allclose(out[check].float(), ref[check], atol=2e-2, rtol=2e-2), (out[check].float() - ref[check]).abs().max()


def test_attention_prefill_sees_a_far_key_and_not_the_future(ops):
    H, KV, D, bs, n = 4, 2, 64, 16, 700
    for far in (0, 17, 255, 256, 640):
        q_unused, k_pages, v_pages, tables, _ = paged_case(BF16, H, KV, D, bs, [n], seed=far, k_scale=0.05)
        q = torch.randn(n, H, D, device=DEV).to(BF16)
        page, off = int(tables[0, far // bs]), far % bs
        k_pages[page, 0, off] = (q[650, 0].float() * 4.0).to(BF16)  # query 650 of head 0 matches key `far`
        fut_page, fut_off = int(tables[0, 651 // bs]), 651 % bs
        k_pages[fut_page, 0, fut_off] = (q[650, 0].float() * 8.0).to(BF16)  # a stronger match, one step in the future
        tiles = [[q0, min(64, n - q0), 0, q0] for q0 in range(0, n, 64)]
        for query_tiles, cut in ((1, 1), (2, 1), (2, 2), (1, 3), (2, 5)):  # cut: the far key lies in one piece, the future one in the last
            out = torch.zeros(n, H, D, dtype=BF16, device=DEV)
            with prefill_cut(ops, cut):
                ops.attn_prefill(q, k_pages, v_pages, i32(tiles), tables, out, 1.0, 0, n, query_tiles=query_tiles)
            assert torch.allclose(out[650, 0].float(), v_pages[page, 0, :, off].float(), atol=2e-2), (far, query_tiles, cut)


class prefill_cut:
    """Within it, `ops.attn_prefill` cuts long work items into that many pieces (1: never; None: as the sizes say)."""

    def __init__(self, ops, pieces):
        self.ops, self.pieces = ops, pieces

    def __enter__(self):
        self.before, self.ops.PREFILL_PIECES = self.ops.PREFILL_PIECES, self.pieces

    def __exit__(self, *exc):
        self.ops.PREFILL_PIECES = self.before


@pytest.mark.parametrize("H,KV,D,bs,n,start,window,pieces", [
    (32, 8, 128, 16, 2048, 0, 0, 2), (16, 8, 128, 16, 1000, 0, 0, 3), (6, 2, 32, 16, 777, 130, 0, 2), (8, 2, 64, 32, 1500, 0, 1000, 4),
    (64, 8, 128, 16, 640, 64, 0, 2), (32, 8, 128, 16, 512, 3584, 0, 4), (32, 8, 128, 16, 200, 9000, 0, 8), (4, 4, 256, 16, 300, 2100, 0, 5)])
def test_long_items_of_a_prompt_step_are_cut_into_pieces_and_merged(ops, H, KV, D, bs, n, start, window, pieces):
    """A step of few work items lasts as long as the longest: items of more rounds than a piece has are cut along
    their keys, the pieces' maxima, sums and outputs merged.  The entry point called as the wrapper calls it, on a
    lone prompt (items of every length: some are cut, in two or more, and some are not) and on a portion behind a
    long prefix (all are): the result is the plain attention's, and the kernel's without the cut."""
    from atomserve_amd.kernels.lib import call

    torch.manual_seed(n + H)
    _, k_pages, v_pages, tables, _ = paged_case(BF16, H, KV, D, bs, [start + n], seed=4, k_scale=2.0 / math.sqrt(D / 16))
    q = torch.randn(n, H, D, device=DEV).to(BF16)
    tiles = sorted(([q0, min(64, n - q0), 0, start + q0] for q0 in range(0, n, 64)), key=lambda t: -(t[3] + t[1]))
    check = sorted({0, 1, min(63, n - 1), min(64, n - 1), n // 2 - 1, n // 2, min(n - 1, n // 2 + 70), max(0, n - 65), n - 2, n - 1} | set(range(5, n, 211)))
    ref = pk.paged_attention(q, k_pages, v_pages, i32(check), i32(list(range(start, start + n))), i32([0] * n), tables, D**-0.5, window)
    stream = torch.cuda.current_stream().cuda_stream
    for query_tiles in (2, 1):
        with prefill_cut(ops, pieces):
            kind, got_pieces, piece_rounds = ops._prefill_plan(len(tiles), H, KV, D, start + n, window, query_tiles)
        span = min(start + n, window + 64) if window else start + n
        assert kind == query_tiles and got_pieces == pieces and piece_rounds == -(-(-(-span // 64)) // pieces)
        units = ops._prefill_units(query_tiles, H // KV)
        cut = torch.full((len(tiles) * KV * units,), -1, dtype=I32, device=DEV)
        part_ml = torch.full((n, H, pieces, 2), float("nan"), device=DEV)
        part_acc = torch.full((n, H, pieces, D), float("nan"), device=DEV)
        out = torch.zeros(n, H, D, dtype=BF16, device=DEV)
        call("as_attn_prefill_mfma", q.data_ptr(), k_pages.data_ptr(), v_pages.data_ptr(), i32(tiles).data_ptr(), len(tiles),
             tables.data_ptr(), tables.shape[1], out.data_ptr(), H, KV, D, bs, D**-0.5, window, query_tiles, pieces, piece_rounds,
             cut.data_ptr(), part_ml.data_ptr(), part_acc.data_ptr(), stream)  # fmt: skip
        said = set(cut.tolist())
        assert said <= set(range(1, pieces + 1)) and pieces in said  # every item said how many pieces it is; the longest all of them
        # (a work item is a tile's queries of some heads: those of a tile may be cut differently, and a tile of fewer
        # than 64 queries leaves some of its workgroups without work)
        full = [i for i, t in enumerate(tiles) if t[1] == 64]
        per_tile = cut.view(len(tiles), -1).float().mean(1)[full]
        assert bool((per_tile[:-1] >= per_tile[1:]).all())  # the more keys an item sees, the more pieces
        if start == 0:
            assert 1 in said and per_tile[-1] == 1  # the first tile of a lone prompt is not cut
        assert torch.allclose(out[check].float(), ref[check], atol=2e-2, rtol=2e-2), (out[check].float() - ref[check]).abs().max()
        whole = torch.zeros(n, H, D, dtype=BF16, device=DEV)
        with prefill_cut(ops, 1):
            ops.attn_prefill(q, k_pages, v_pages, i32(tiles), tables, whole, D**-0.5, window, start + n, query_tiles=query_tiles)
        assert torch.allclose(out.float(), whole.float(), atol=2e-2, rtol=2e-2)  # every token, against the kernel without the cut


def test_kernels_refuse_what_they_cannot_do(ops):
    from atomserve_amd.kernels.lib import KernelError

    x = torch.zeros(2, 8, device=DEV)
    with pytest.raises(KernelError):
        ops.rmsnorm(x, torch.ones(9, device=DEV), 1e-6, torch.empty_like(x))
    with pytest.raises(KernelError):
        ops.rmsnorm(x.cpu(), torch.ones(8), 1e-6, torch.empty(2, 8))
    q = torch.zeros(1, 2, 6, device=DEV)
    with pytest.raises(KernelError, match="head width"):
        ops.attn_single_query(q, torch.zeros(1, 1, 4, 6, device=DEV), torch.zeros(1, 1, 6, 4, device=DEV), i32([0]),
                              i32([0]), i32([0]), i32([[0]]), torch.zeros_like(q), 1.0, 0, 1)  # fmt: skip


# ---- sampling -------------------------------------------------------------------------


def test_argmax_and_ties(ops):
    torch.manual_seed(9)
    logits = torch.randn(7, 151936, device=DEV) * 4
    out = torch.empty(7, dtype=I32, device=DEV)
    ops.argmax(logits, out)
    assert out.tolist() == logits.argmax(dim=-1).tolist()
    ties = torch.zeros(2, 1000, device=DEV)
    ties[0, [17, 400]] = 3.0
    ties[1, :] = float("-inf")
    ties[1, 999] = -5.0
    out = torch.empty(2, dtype=I32, device=DEV)
    ops.argmax(ties, out)
    assert out.tolist() == [17, 999]


def test_topk_matches_the_library(ops):
    """Exact values for every k, with heavy ties and rows with fewer finite entries than k
    (cases of reference tests/test_kernels.py:155-171)."""
    torch.manual_seed(10)
    cases = [
        torch.randn(7, 151936, device=DEV) * 4,
        torch.randint(-5, 5, (3, 151936), device=DEV).float(),
        torch.full((2, 151936), float("-inf"), device=DEV).index_fill_(1, torch.tensor([3, 9], device=DEV), 1.0),
    ]
    for x in cases:
        for k in (1, 2, 20, 33, 64):
            values = torch.empty(x.shape[0], k, device=DEV)
            indices = torch.empty(x.shape[0], k, dtype=I32, device=DEV)
            ops.topk(x, k, values, indices)
            expected = pk.topk_values(x, k)
            assert torch.equal(values, expected)
            assert torch.equal(x.gather(1, indices.long().clamp_min(0)), expected)


def sample_rows(ops, logits, temperature, top_k, top_p, seeds, counters=None, max_top_k=None):
    B = logits.shape[0]
    out = torch.empty(B, dtype=I32, device=DEV)
    f = lambda v: torch.full((B,), v, dtype=F32, device=DEV) if not torch.is_tensor(v) else v  # noqa: E731
    ops.sample(logits, f(temperature), torch.full((B,), top_k, dtype=I32, device=DEV) if not torch.is_tensor(top_k) else top_k,
               f(top_p), torch.as_tensor(seeds, dtype=torch.int64).to(DEV),
               torch.zeros(B, dtype=I32, device=DEV) if counters is None else counters, out, max_top_k=max_top_k)  # fmt: skip
    return out


PROBS = torch.tensor([0.4, 0.3, 0.2, 0.1])


def test_sampling_follows_the_distribution(ops):
    """Frequencies over 20,000 draws (reference tests/test_sampler.py:33-47), through the
    top-k path and through the all-tokens path."""
    n = 20000
    logits = PROBS.log().repeat(n, 1).to(DEV)
    seeds = torch.arange(n) * 7919 + 1
    for top_k in (0, 3):
        draws = sample_rows(ops, logits, 1.0, top_k, 1.0, seeds)
        freq = draws.long().bincount(minlength=4).float().cpu() / n
        want = PROBS if top_k == 0 else torch.tensor([0.4, 0.3, 0.2, 0.0]) / 0.9
        assert torch.allclose(freq, want, atol=0.015), (top_k, freq)
    assert set(sample_rows(ops, logits[:2000], 1.0, 2, 1.0, seeds[:2000]).tolist()) == {0, 1}
    assert set(sample_rows(ops, logits[:200], 1.0, 1, 1.0, seeds[:200]).tolist()) == {0}
    for top_k in (0, 4):  # top-p through both paths
        assert set(sample_rows(ops, logits[:2000], 1.0, top_k, 0.6, seeds[:2000]).tolist()) == {0, 1}
        assert set(sample_rows(ops, logits[:200], 1.0, top_k, 0.01, seeds[:200]).tolist()) == {0}
    sharp = sample_rows(ops, logits, 0.5, 0, 1.0, seeds).long().bincount(minlength=4).float().cpu() / n
    assert torch.allclose(sharp, PROBS**2 / (PROBS**2).sum(), atol=0.015)


@pytest.mark.parametrize("V", [151936, 4097, 100, 31])
def test_sampling_split_over_workgroups_draws_the_same_tokens(ops, V):
    """Rows that keep few candidates are searched by many workgroups: the same tokens as the
    one-workgroup kernel, also among equal logits (the lower index ranks first), with greedy
    rows, every top-p and fewer tokens than slices."""
    torch.manual_seed(14)
    B = 24
    logits = torch.randn(B, V, device=DEV) * 3
    logits[B // 2 :] = (logits[B // 2 :] * 2).round() / 2  # long runs of equal values
    logits[3, V // 3] = float("nan")
    top_k = i32([(1, 2, 20, 33, 64)[i % 5] if (1, 2, 20, 33, 64)[i % 5] < V else V - 1 for i in range(B)])
    temperature = torch.tensor([(1.0, 0.6, 0.0, 1.5)[i % 4] for i in range(B)], device=DEV)
    top_p = torch.tensor([(1.0, 0.95, 0.5, 0.0, 0.01)[i % 5] for i in range(B)], device=DEV)
    seeds = torch.arange(B) * 104729 + 5
    for c in range(4):
        counters = i32([c] * B)
        one = sample_rows(ops, logits, temperature, top_k, top_p, seeds, counters)
        many = sample_rows(ops, logits, temperature, top_k, top_p, seeds, counters, max_top_k=64)
        assert torch.equal(one, many)


def test_sampling_is_seeded_per_request_and_mixes_greedy_rows(ops):
    torch.manual_seed(11)
    row = torch.randn(1, 1000, device=DEV)
    alone = [int(sample_rows(ops, row, 1.0, 50, 1.0, [7], i32([c]))[0]) for c in range(20)]
    crowd = []
    for c in range(20):
        logits = torch.cat([torch.randn(1, 1000, device=DEV), row, torch.randn(1, 1000, device=DEV)])
        t = torch.tensor([0.8, 1.0, 0.0], device=DEV)
        k = i32([500, 50, 20])
        out = sample_rows(ops, logits, t, k, torch.tensor([0.9, 1.0, 0.95], device=DEV), [3, 7, 5], i32([c, c, c]))
        crowd.append(int(out[1]))
        assert int(out[2]) == int(logits[2].argmax())  # the greedy row is its argmax
    assert alone == crowd and len(set(alone)) > 1


@pytest.mark.parametrize("M,N,K", [(17, 96, 256), (33, 1000, 512), (64, 4096, 1024), (48, 520, 768), (20, 64, 3072), (64, 12, 256),
                                   (65, 200, 512), (96, 1000, 768), (100, 520, 1024), (128, 4096, 256), (81, 36, 1280), (80, 160, 512),
                                   (33, 48, 1024),
                                   # 9 to 16 rows, the one row tile that decode steps of wide models take: a row tile that is
                                   # partly filled, and the widths K of models 2,560, 9,728 and 17,408 wide
                                   (9, 96, 256), (12, 1000, 512), (16, 4096, 1024), (13, 520, 768), (9, 1024, 2560), (12, 2560, 9728),
                                   (16, 5120, 17408), (15, 36, 1280), (10, 64, 3072), (16, 12, 256), (11, 9728, 2560)])  # fmt: skip
def test_products_of_9_to_128_rows_in_tiles(ops, M, N, K):
    """The tile kernel behind `gemm_silu_mul` and `gemm_split`: every tile width (8, 6, 4 and 2 strips),
    plain, gated and with K cut into ranges, against the matrix product in float64; rows and columns that
    do not fill the last tile, chunk counts that are no multiple of three; one row tile (9 to 16 rows, which
    decode steps of wide models take), two, four, and the row tiles of 96 and 128."""
    from atomserve_amd.kernels.lib import call

    torch.manual_seed(M + N)
    a = (torch.randn(M, K, device=DEV) * 0.5).to(BF16)
    w = (torch.randn(2 * N, K, device=DEV) * 0.1).to(BF16)
    stream = torch.cuda.current_stream().cuda_stream
    ref = a.double() @ w.double().T
    gated_ref = (lambda g: torch.nn.functional.silu(g[:, :N]) * g[:, N:])(ref.to(BF16).double())
    chunks = K // 256
    typical = float(ref.pow(2).mean().sqrt())
    copy = ops.Streamed(w).wave if N % 16 == 0 else None  # the gated and the split variant also read weights in wave order
    for strips, wt in [(n, p) for n in (8, 6, 4, 2) for p in ([0] if copy is None else [0, copy.data_ptr()])]:
        out = torch.full((M, N), float("nan"), dtype=BF16, device=DEV)
        call("as_gemm_bf16_tile", a.data_ptr(), w.data_ptr(), wt, out.data_ptr(), 0, 1, M, N, K, 0, 0, strips, stream)
        # one rounding step of bfloat16, and for sums near zero what adding K products in float32 loses
        # (2^-16 of a typical sum; at K = 17,408 a sum of 1e-3 is off by 5e-6 before it is rounded)
        assert close_bf16(out, ref[:, :N], scale=typical * 2.0**-8), f"plain, {strips} strips"
        out32 = torch.full((M, N), float("nan"), dtype=F32, device=DEV)
        call("as_gemm_bf16_tile", a.data_ptr(), w.data_ptr(), wt, out32.data_ptr(), 0, 0, M, N, K, 0, 0, strips, stream)
        assert torch.allclose(out32.double(), ref[:, :N], atol=1e-3, rtol=1e-4)
        assert torch.equal(out, out32.to(BF16))  # the same sums in the same order, rounded once
        out.fill_(float("nan"))
        call("as_gemm_bf16_tile", a.data_ptr(), w.data_ptr(), wt, out.data_ptr(), 0, 1, M, N, K, 1, 0, strips, stream)
        # a sum that rounds to the neighbouring bfloat16 moves the activation by a step of its input
        assert torch.allclose(out.double(), gated_ref, atol=2e-2, rtol=2e-2), f"gated, {strips} strips"
        for splits in sorted({1, 2, 3, chunks, max(1, chunks // 2), max(1, chunks - 1)}):
            if splits > chunks:
                continue
            sums = torch.full((splits, M, N), float("nan"), dtype=F32, device=DEV)
            run = lambda: call("as_gemm_bf16_tile", a.data_ptr(), w.data_ptr(), wt, 0, sums.data_ptr(), 0, M, N, K, 0, splits, strips, stream)
            if (splits - 1) * -(-chunks // splits) >= chunks:  # ranges of ceil(chunks / splits) chunks would leave the last ones empty
                with pytest.raises(ops.KernelError):
                    run()
                continue
            run()  # ranges of equal length, or the last one shorter
            assert torch.allclose(sums.double().sum(0), ref[:, :N], atol=1e-3, rtol=1e-4), f"{splits} ranges, {strips} strips"
    # through the wrappers: the gated product, and split sums taken in by the norm
    for weights in (w, ops.Streamed(w)):  # from rows, and from the copy in wave order where the sizes allow one
        act = torch.full((M, N), float("nan"), dtype=BF16, device=DEV)
        ops.gemm_silu_mul(a, weights, act)
        assert torch.allclose(act.double(), gated_ref, atol=2e-2, rtol=2e-2)
    if N % 4 == 0:
        sums = ops.gemm_split(a, ops.Streamed(w[:N].contiguous()))
        assert torch.equal(sums, ops.gemm_split(a, w[:N].contiguous()))  # the same values reach the same lanes
        x = torch.randn(M, N, device=DEV)
        gain = (torch.randn(N, device=DEV) + 1).to(BF16)
        x1, x2 = x.clone(), x.clone()
        out1, out2 = torch.empty(M, N, dtype=BF16, device=DEV), torch.empty(M, N, dtype=BF16, device=DEV)
        ops.rmsnorm(x1, gain, 1e-5, out1, split_sums=sums)
        total = sums[0].clone()
        for part in sums[1:]:  # in the order of the ranges, as the norm adds them: the same float32 sum, bit for bit
            total += part
        delta = total.to(BF16)
        ops.rmsnorm(x2, gain, 1e-5, out2, delta=delta)
        assert torch.equal(x1, x2) and close_bf16(out1, out2.double())
        rows = i32([M - 1, 0, 3])
        sel = torch.empty(3, N, dtype=BF16, device=DEV)
        x3 = x.clone()
        ops.rmsnorm(x3, gain, 1e-5, sel, rows=rows, update_x=False, split_sums=sums)
        assert torch.equal(x3, x) and close_bf16(sel, out2[[M - 1, 0, 3]].double())
