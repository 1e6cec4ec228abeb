"""Each HIP kernel alone against its plain torch twin, at sizes other than the tiny models'."""

import math

import pytest
import torch

from twins import TwinKernels

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def hip():
    from simple_inference_amd.kernels import HipKernels
    return HipKernels()


twin = TwinKernels()


def tol(dtype):
    return dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1.6e-2, atol=1e-2)


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


class Ctx:
    """The fields of a step context that the kernels read."""

    def __init__(self, q_lens, kv_lens):
        pos, sot, cu = [], [], [0]
        for s, (q, kv) in enumerate(zip(q_lens, kv_lens)):
            pos += list(range(kv - q, kv))
            sot += [s] * q
            cu.append(cu[-1] + q)
        i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
        self.positions, self.seq_of_token, self.cu_q, self.kv_len = i32(pos), i32(sot), i32(cu), i32(kv_lens)
        self.n_tokens, self.n_seqs = len(pos), len(q_lens)
        self.max_q_len, self.max_kv_len = max(q_lens), max(kv_lens)
        self.q_lens, self.kv_bound = list(q_lens), 0
        self.n_decode_seqs = next((i for i, q in enumerate(q_lens) if q != 1), len(q_lens))


class Cache:
    def __init__(self, n_pages, n_kv, page_size, head_dim, dtype, kv_lens, seed=0):
        self.page_size = page_size
        self.k_pages = torch.zeros(n_pages, n_kv, page_size, head_dim, dtype=dtype, device=DEV)
        self.v_pages = torch.zeros(n_pages, n_kv, head_dim, page_size, dtype=dtype, device=DEV)
        g = torch.Generator().manual_seed(seed)
        perm = torch.randperm(n_pages, generator=g).tolist()  # pages in no particular order
        width = max(-(-kv // page_size) for kv in kv_lens)
        table = torch.full((len(kv_lens), width), -1, dtype=torch.int32)
        for s, kv in enumerate(kv_lens):
            for i in range(-(-kv // page_size)):
                table[s, i] = perm.pop()
        self.block_table = table.to(DEV)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [72, 1000, 3072])
def test_embed(hip, dtype, hidden):
    table = rnd(517, hidden, dtype=dtype)
    ids = torch.tensor([0, 516, 3, 3, 100], dtype=torch.int32, device=DEV)
    assert torch.equal(hip.embed(ids, table), twin.embed(ids, table))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [40, 1000, 3072, 5000])
def test_add_rmsnorm(hip, dtype, hidden):
    res = rnd(7, hidden, seed=1, scale=3.0)
    delta = rnd(7, hidden, dtype=dtype, seed=2)
    w = 1 + 0.1 * rnd(hidden, seed=3)
    r1, r2 = res.clone(), res.clone()
    out = hip.add_rmsnorm(r1, delta, w, 1e-5, dtype)
    ref = twin.add_rmsnorm(r2, delta, w, 1e-5, dtype)
    torch.testing.assert_close(out.float(), ref.float(), **tol(dtype))
    torch.testing.assert_close(r1, r2, rtol=0, atol=0)
    # no delta; selected rows leave the residual alone
    rows = torch.tensor([6, 0, 3], dtype=torch.int32, device=DEV)
    r3 = res.clone()
    out = hip.add_rmsnorm(r3, delta, w, 1e-5, dtype, rows)
    ref = twin.add_rmsnorm(res.clone(), delta, w, 1e-5, dtype, rows)
    torch.testing.assert_close(out.float(), ref.float(), **tol(dtype))
    assert torch.equal(r3, res)
    out = hip.add_rmsnorm(r3, None, w, 1e-5, dtype)
    torch.testing.assert_close(out.float(), twin.add_rmsnorm(res.clone(), None, w, 1e-5, dtype).float(), **tol(dtype))


def test_rmsnorm_eps_is_inside_the_root(hip):
    x = torch.full((1, 64), 1e-4, device=DEV)
    w = torch.ones(64, device=DEV)
    out = hip.add_rmsnorm(x.clone(), None, w, 1e-2, torch.float32)
    assert abs(out[0, 0].item() - 1e-4 / math.sqrt(1e-8 + 1e-2)) < 1e-8


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inter", [24, 37, 1000, 8192])
def test_swiglu(hip, dtype, inter):
    gu = rnd(5, 2 * inter, dtype=dtype, scale=3.0)
    torch.testing.assert_close(hip.swiglu(gu).float(), twin.swiglu(gu).float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(1, 37, 50), (5, 130, 77), (70, 64, 256), (130, 3, 1000)])
def test_gemm_generic(hip, dtype, shape):
    M, N, K = shape
    x, w = rnd(M, K, dtype=dtype, seed=1), rnd(N, K, dtype=dtype, seed=2)
    ref = x.double() @ w.double().T
    out = hip.gemm_generic(x, w, out_float32=True)
    torch.testing.assert_close(out.double(), ref, rtol=1e-5, atol=1e-4)
    if dtype == torch.bfloat16:
        out = hip.gemm_generic(x, w)
        assert out.dtype == torch.bfloat16
        torch.testing.assert_close(out.double(), ref, **tol(dtype))


@pytest.mark.parametrize("shape", [(1, 48, 64), (8, 5120, 3072), (16, 3072, 8192), (3, 16, 320), (11, 1008, 1024),
                                   (7, 203, 192), (2, 1, 64), (9, 4099, 128), (16, 16384, 576)])
def test_gemm_skinny(hip, shape):
    """bfloat16 products with few rows: this package's kernel against a float64 product and the library."""
    M, N, K = shape
    x, w = rnd(M, K, dtype=torch.bfloat16, seed=1), rnd(N, K, dtype=torch.bfloat16, seed=2)
    ref = x.double() @ w.double().T
    out = hip.linear(x, w, out_float32=True)
    assert out.dtype == torch.float32
    torch.testing.assert_close(out.double(), ref, rtol=1e-4, atol=1e-3 * math.sqrt(K / 64))
    out16 = hip.linear(x, w)
    assert out16.dtype == torch.bfloat16
    torch.testing.assert_close(out16.double(), ref, rtol=1e-2, atol=1e-2 * math.sqrt(K / 64))
    hip.use_skinny_gemm = False
    try:
        lib = hip.linear(x, w)
    finally:
        hip.use_skinny_gemm = True
    torch.testing.assert_close(out16.float(), lib.float(), rtol=2e-2, atol=2e-2 * math.sqrt(K / 64))
    # a row's result does not depend on the other rows
    assert torch.equal(hip.linear(x[:1].contiguous(), w), out16[:1])


@pytest.mark.parametrize("shape", [(1, 32, 64), (8, 8192, 3072), (16, 1008, 512), (5, 96, 320), (40, 128, 256),
                                   (3, 1, 64), (12, 333, 192), (16, 14336, 256)])
def test_gated_linear(hip, shape):
    """The product with the SwiGLU activation in its epilogue (few rows) or after it, against the twin."""
    M, inter, K = shape
    x = rnd(M, K, dtype=torch.bfloat16, seed=1)
    w = rnd(2 * inter, K, dtype=torch.bfloat16, seed=2, scale=1 / math.sqrt(K))
    gu = x.double() @ w.double().T
    ref = torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]
    out = hip.gated_linear(x, w)
    assert out.shape == (M, inter) and out.dtype == torch.bfloat16
    torch.testing.assert_close(out.double(), ref, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("shape", [(17, 3072, 3072), (512, 5120, 3072), (2048, 16384, 3072), (130, 3072, 8192),
                                   (33, 1008, 200), (64, 320, 96)])
def test_library_product_called_directly(hip, shape):
    """Products of many rows go to the BLAS library without a tensor library between: same results as through torch
    (it is the same library), against a float64 product, bfloat16 and float results, again on a second call (the
    kept algorithm)."""
    M, N, K = shape
    assert hip.blas is not None, "the direct way to the BLAS library was not built or did not initialise"
    x, w = rnd(M, K, dtype=torch.bfloat16, seed=1), rnd(N, K, dtype=torch.bfloat16, seed=2)
    ref = x.double() @ w.double().T
    for _ in range(2):
        out = hip.linear(x, w)
        assert out.dtype == torch.bfloat16
        torch.testing.assert_close(out.double(), ref, rtol=1e-2, atol=1e-2 * math.sqrt(K / 64))
        torch.testing.assert_close(out.float(), torch.mm(x, w.t()).float(), rtol=2e-2, atol=2e-2 * math.sqrt(K / 64))
        wide = hip.linear(x, w, out_float32=True)
        assert wide.dtype == torch.float32
        torch.testing.assert_close(wide.double(), ref, rtol=1e-2, atol=1e-2 * math.sqrt(K / 64))


@pytest.mark.parametrize("shape", [(64, 3072, 3072), (33, 1008, 200), (256, 320, 512), (300, 128, 64)])
def test_library_product_with_candidates_tried_out(hip, shape):
    """Inside ``recurring_shapes`` the library's candidate algorithms are timed on the call's own operands and one is
    kept: the product is right on that call and on those after it, inside and outside, also for a shape that had an
    algorithm before."""
    M, N, K = shape
    assert hip.blas is not None
    x, w = rnd(M, K, dtype=torch.bfloat16, seed=3), rnd(N, K, dtype=torch.bfloat16, seed=4)
    ref = x.double() @ w.double().T
    outs = [hip.linear(x, w)]
    with hip.recurring_shapes():
        outs += [hip.linear(x, w), hip.linear(x, w, out_float32=True)]
    outs += [hip.linear(x, w)]
    for out in outs:
        torch.testing.assert_close(out.double(), ref, rtol=1e-2, atol=1e-2 * math.sqrt(K / 64))
    assert torch.equal(outs[1], outs[3])   # the kept algorithm is used from then on


def test_float32_product_has_no_reduced_precision(hip):
    """An operand bit below bfloat16 (8 bits) and tf32 (10 bits) resolution must reach the product."""
    K = 8
    x = torch.ones(1, K, device=DEV)
    w = torch.ones(2, K, device=DEV)
    w[1, 3] += 2.0 ** -12
    y = hip.linear(x, w)
    assert y.dtype == torch.float32
    assert y[0, 0].item() == 8.0
    assert y[0, 1].item() - 8.0 == 2.0 ** -12


def test_linear_rows_do_not_depend_on_the_batch(hip):
    x, w = rnd(67, 300, seed=1), rnd(130, 300, seed=2)
    whole = hip.linear(x, w)
    assert torch.equal(whole[13:14], hip.linear(x[13:14].contiguous(), w))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [
    # heads, kv heads, head_dim, rotary_dim, page_size
    (4, 2, 16, 16, 4), (3, 1, 32, 32, 8), (6, 3, 80, 80, 16), (8, 8, 128, 64, 32), (2, 1, 256, 256, 64),
    (5, 5, 48, 0, 2),
])
def test_rope_kv_write_and_attention(hip, dtype, geom):
    n_heads, n_kv, D, rd, ps = geom
    q_lens, kv_lens = [1, 7, 64, 3], [130, 7, 64 + 37, 66]
    ctx = Ctx(q_lens, kv_lens)
    pages = sum(-(-kv // ps) for kv in kv_lens) + 3
    c_hip = Cache(pages, n_kv, ps, D, dtype, kv_lens, seed=4)
    c_twin = Cache(pages, n_kv, ps, D, dtype, kv_lens, seed=4)
    # earlier tokens' keys and values already in the pages (same in both)
    c_hip.k_pages.copy_(rnd(*c_hip.k_pages.shape, dtype=dtype, seed=5)); c_twin.k_pages.copy_(c_hip.k_pages)
    c_hip.v_pages.copy_(rnd(*c_hip.v_pages.shape, dtype=dtype, seed=6)); c_twin.v_pages.copy_(c_hip.v_pages)
    qkv = rnd(ctx.n_tokens, (n_heads + 2 * n_kv) * D, dtype=dtype, seed=7)
    q1, q2 = qkv.clone(), qkv.clone()
    pos = torch.arange(256, dtype=torch.float32)
    inv = 1.0 / (10000.0 ** (torch.arange(0, max(rd, 2), 2, dtype=torch.float32) / max(rd, 2)))
    ang = torch.outer(pos, inv)
    cos, sin = ang.cos().to(DEV), ang.sin().to(DEV)
    hip.rope_kv_write(q1, n_heads, n_kv, D, rd, cos, sin, ctx, c_hip)
    twin.rope_kv_write(q2, n_heads, n_kv, D, rd, cos, sin, ctx, c_twin)
    torch.testing.assert_close(q1.float(), q2.float(), **tol(dtype))
    torch.testing.assert_close(c_hip.k_pages.float(), c_twin.k_pages.float(), **tol(dtype))
    assert torch.equal(c_hip.v_pages, c_twin.v_pages)
    for window in (None, 19):
        out = hip.paged_attention(q2, n_heads, n_kv, D, 1 / math.sqrt(D), window, ctx, c_twin)
        ref = twin.paged_attention(q2, n_heads, n_kv, D, 1 / math.sqrt(D), window, ctx, c_twin)
        torch.testing.assert_close(out.float(), ref.float(), **tol(dtype))


@pytest.mark.parametrize("geom", [(24, 8, 128, 128, 16), (5, 1, 48, 32, 8), (3, 3, 64, 64, 4)])
def test_rope_kv_write_of_a_long_step(hip, geom):
    """More than a thousand tokens in one step (the kernel then gives a thread several items): two prompt portions,
    one from the start of its sequence and one that begins in the middle of a page, and a single decoded token."""
    n_heads, n_kv, D, rd, ps = geom
    q_lens, kv_lens = [1, 700, 450], [77, 700, 450 + 21]
    ctx = Ctx(q_lens, kv_lens)
    pages = sum(-(-kv // ps) for kv in kv_lens) + 2
    c_hip = Cache(pages, n_kv, ps, D, torch.bfloat16, kv_lens, seed=14)
    c_twin = Cache(pages, n_kv, ps, D, torch.bfloat16, kv_lens, seed=14)
    c_hip.k_pages.copy_(rnd(*c_hip.k_pages.shape, dtype=torch.bfloat16, seed=15)); c_twin.k_pages.copy_(c_hip.k_pages)
    c_hip.v_pages.copy_(rnd(*c_hip.v_pages.shape, dtype=torch.bfloat16, seed=16)); c_twin.v_pages.copy_(c_hip.v_pages)
    qkv = rnd(ctx.n_tokens, (n_heads + 2 * n_kv) * D, dtype=torch.bfloat16, seed=17)
    q1, q2 = qkv.clone(), qkv.clone()
    ang = torch.outer(torch.arange(720, dtype=torch.float32), 1.0 / (500000.0 ** (torch.arange(0, rd, 2, dtype=torch.float32) / rd)))
    cos, sin = ang.cos().to(DEV), ang.sin().to(DEV)
    hip.rope_kv_write(q1, n_heads, n_kv, D, rd, cos, sin, ctx, c_hip)
    twin.rope_kv_write(q2, n_heads, n_kv, D, rd, cos, sin, ctx, c_twin)
    torch.testing.assert_close(q1.float(), q2.float(), **tol(torch.bfloat16))
    torch.testing.assert_close(c_hip.k_pages.float(), c_twin.k_pages.float(), **tol(torch.bfloat16))
    assert torch.equal(c_hip.v_pages, c_twin.v_pages)


@pytest.mark.parametrize("geom", [
    # heads, kv heads, head_dim, page_size, hidden, rows
    (24, 8, 128, 64, 3072, 8), (3, 1, 32, 8, 192, 16), (5, 5, 96, 16, 1088, 1), (2, 1, 256, 32, 64, 5),
    (7, 7, 64, 4, 2048, 13), (5, 1, 48, 16, 320, 9), (32, 8, 64, 16, 2048, 4), (1, 1, 16, 2, 64, 3),
])
def test_qkv_product_that_rotates_and_writes_the_pages(hip, geom):
    """Few rows: one kernel multiplies, rotates q and k and writes k and v into the pages.  Compared with the
    product, rotation and write done one after the other on float sums (the twin rounds the product first, so
    its result is a rounding away)."""
    n_heads, n_kv, D, ps, hidden, rows = geom
    dtype = torch.bfloat16
    kv_lens = [3 + 41 * i for i in range(rows)]
    kv_lens[-1] = 2 * ps  # a token in the last slot of a page
    if rows > 1:
        kv_lens[0] = ps + 1  # and one in the first
    ctx = Ctx([1] * rows, kv_lens)
    pages = sum(-(-kv // ps) for kv in kv_lens) + 3
    c_hip = Cache(pages, n_kv, ps, D, dtype, kv_lens, seed=4)
    c_ref = Cache(pages, n_kv, ps, D, torch.float32, kv_lens, seed=4)  # float pages: rounded once, at the comparison
    c_hip.k_pages.copy_(rnd(*c_hip.k_pages.shape, dtype=dtype, seed=5)); c_ref.k_pages.copy_(c_hip.k_pages)
    c_hip.v_pages.copy_(rnd(*c_hip.v_pages.shape, dtype=dtype, seed=6)); c_ref.v_pages.copy_(c_hip.v_pages)
    x = rnd(rows, hidden, dtype=dtype, seed=7)
    w = rnd((n_heads + 2 * n_kv) * D, hidden, dtype=dtype, seed=8, scale=hidden ** -0.5)
    pos = torch.arange(max(kv_lens) + 1, dtype=torch.float32)
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    ang = torch.outer(pos, inv)
    cos, sin = ang.cos().to(DEV), ang.sin().to(DEV)
    launched = []
    real = hip.core.sia_gemm_skinny_rope
    hip.core.sia_gemm_skinny_rope = lambda *a: launched.append(1) or real(*a)
    try:
        qkv = hip.qkv_to_cache(x, w, n_heads, n_kv, D, D, cos, sin, ctx, c_hip)
    finally:
        hip.core.sia_gemm_skinny_rope = real
    assert launched, "the fused kernel did not run"
    # reference: float product, rotated in float, rounded once
    ref = (x.float() @ w.float().T)
    twin.rope_kv_write(ref, n_heads, n_kv, D, D, cos, sin, ctx, c_ref)
    nq = n_heads * D
    torch.testing.assert_close(qkv[:, :nq].float(), ref[:, :nq], **tol(dtype))
    torch.testing.assert_close(c_hip.k_pages.float(), c_ref.k_pages, **tol(dtype))
    torch.testing.assert_close(c_hip.v_pages.float(), c_ref.v_pages, **tol(dtype))
    # nothing but the tokens' own slots has changed
    before = rnd(*c_hip.k_pages.shape, dtype=dtype, seed=5)
    changed = (c_hip.k_pages != before).any(dim=-1)            # [page, kv head, offset]
    assert int(changed.any(dim=1).sum()) <= rows
    # and the separate path gives the same within the rounding of the product
    qkv2 = hip.linear(x, w)
    c_two = Cache(pages, n_kv, ps, D, dtype, kv_lens, seed=4)
    c_two.k_pages.copy_(before); c_two.v_pages.copy_(rnd(*c_hip.v_pages.shape, dtype=dtype, seed=6))
    hip.rope_kv_write(qkv2, n_heads, n_kv, D, D, cos, sin, ctx, c_two)
    torch.testing.assert_close(qkv[:, :nq].float(), qkv2[:, :nq].float(), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(c_hip.k_pages.float(), c_two.k_pages.float(), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(c_hip.v_pages.float(), c_two.v_pages.float(), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("shape", [
    # rows, hidden, inner (the K of the product into the residual), intermediate of the gated product after it
    (8, 3072, 8192, 8192), (1, 3072, 3072, 8192), (16, 192, 64, 96), (5, 5120, 1024, 5120), (13, 1088, 2048, 320),
    (4, 4160, 128, 1001), (16, 4096, 14336, 1024),
])
def test_norm_shared_out_between_the_products_around_it(hip, shape):
    """Few rows: the product before a norm adds into the residual and leaves gain * x and sums of squares; the product
    after it divides its rows by the root mean square.  Compared with product, add + norm and product one by one."""
    from simple_inference_amd.kernels import PendingProduct, ScaledRows
    rows, hidden, inner, inter = shape
    eps = 1e-5
    x = rnd(rows, inner, dtype=torch.bfloat16, seed=1)
    w = rnd(hidden, inner, dtype=torch.bfloat16, seed=2, scale=inner ** -0.5)
    res = rnd(rows, hidden, seed=3, scale=3.0)
    res[0] *= 40.0   # rows of very different size: each needs its own scale
    gain = (rnd(hidden, seed=4, scale=0.3) + 1.0).contiguous()
    w_gu = rnd(2 * inter, hidden, dtype=torch.bfloat16, seed=5, scale=hidden ** -0.5)

    pending = hip.pending_linear(x, w)
    assert isinstance(pending, PendingProduct)
    res_fused = res.clone()
    scaled = hip.linear_into_residual(pending, res_fused, gain, eps)
    assert isinstance(scaled, ScaledRows)

    res_plain = res.clone()
    normed = hip.add_rmsnorm(res_plain, hip.linear(x, w), gain, eps, torch.bfloat16, None)
    # the residual: same sum unless the plain product went to the library, then a rounding of the delta apart
    torch.testing.assert_close(res_fused, res_plain, rtol=0, atol=2 ** -7)
    want = res.double() + (x.double() @ w.double().T)
    torch.testing.assert_close(res_fused.double(), want, rtol=0, atol=2 ** -6)
    # what it leaves for the product after it: gain * x rounded once, and the sums of squares
    assert torch.equal(scaled.rows, (res_fused * gain).to(torch.bfloat16))
    assert scaled.partials.shape[1] == 16 and hidden / 16 <= scaled.partials.shape[0] <= hidden / 8 + 4   # blocks of 8 to 16 columns
    sums = scaled.partials[:, :rows].double().sum(0)
    torch.testing.assert_close(sums, res_fused.double().pow(2).sum(-1), rtol=1e-5, atol=0)
    rs = torch.rsqrt(sums / hidden + eps)[:, None]
    normed_rows = scaled.rows.double() * rs   # the rows that the fused products multiply, exactly
    torch.testing.assert_close(hip.finish_rows(scaled).double(), normed_rows, **tol(torch.bfloat16))
    torch.testing.assert_close(normed.double(), normed_rows, **tol(torch.bfloat16))

    def mean_error(got, ref):
        return float((got.double() - ref).abs().mean())

    # the gated product: exact given the rows it multiplies, and as near the exact norm as the plain path is
    gu = normed_rows @ w_gu.double().T
    fused = hip.gated_linear(scaled, w_gu)
    torch.testing.assert_close(fused.double(), torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:],
                               **tol(torch.bfloat16))
    exact = want * torch.rsqrt(want.pow(2).mean(-1, keepdim=True) + eps) * gain.double()
    gu = exact @ w_gu.double().T
    ref = torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]
    assert mean_error(fused, ref) <= 1.25 * mean_error(hip.gated_linear(normed, w_gu), ref) + 1e-5
    torch.testing.assert_close(hip.linear(scaled, w_gu).double(), normed_rows @ w_gu.double().T, **tol(torch.bfloat16))

    # and into the q/k/v product that rotates and writes the pages
    D, n_kv, ps = 32, 2, 16
    n_heads = 4
    w_qkv = rnd((n_heads + 2 * n_kv) * D, hidden, dtype=torch.bfloat16, seed=6, scale=hidden ** -0.5)
    kv_lens = [7 + 19 * i for i in range(rows)]
    ctx = Ctx([1] * rows, kv_lens)
    pages = sum(-(-kv // ps) for kv in kv_lens) + 2
    c1 = Cache(pages, n_kv, ps, D, torch.bfloat16, kv_lens, seed=4)
    c2 = Cache(pages, n_kv, ps, D, torch.float32, kv_lens, seed=4)
    ang = torch.outer(torch.arange(max(kv_lens) + 1, dtype=torch.float32),
                      1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D)))
    cos, sin = ang.cos().to(DEV), ang.sin().to(DEV)
    q1 = hip.qkv_to_cache(scaled, w_qkv, n_heads, n_kv, D, D, cos, sin, ctx, c1)
    q2 = (normed_rows @ w_qkv.double().T).float()
    twin.rope_kv_write(q2, n_heads, n_kv, D, D, cos, sin, ctx, c2)
    torch.testing.assert_close(q1[:, :n_heads * D].float(), q2[:, :n_heads * D], **tol(torch.bfloat16))
    torch.testing.assert_close(c1.k_pages.float(), c2.k_pages, **tol(torch.bfloat16))
    torch.testing.assert_close(c1.v_pages.float(), c2.v_pages, **tol(torch.bfloat16))


@pytest.mark.parametrize("geom", [
    # heads, kv heads, head_dim, page_size, window
    (24, 8, 128, 16, None), (32, 8, 64, 64, None), (16, 1, 32, 8, None), (6, 2, 48, 16, 100), (5, 5, 112, 32, 700),
    (34, 2, 16, 16, None),
])
def test_matrix_core_attention_decode_and_mixed(hip, geom):
    """Many single-token sequences of different lengths (so that splits differ), alone and beside longer runs."""
    n_heads, n_kv, D, ps, window = geom
    dtype = torch.bfloat16
    for q_lens, kv_lens in (([1] * 7, [1, 63, 64, 65, 300, 1027, 2500]),
                            ([1, 1, 1, 130, 5, 257], [513, 17, 2048, 130, 900, 300])):
        ctx = Ctx(q_lens, kv_lens)
        pages = sum(-(-kv // ps) for kv in kv_lens) + 5
        cache = Cache(pages, n_kv, ps, D, dtype, kv_lens, seed=8)
        cache.k_pages.copy_(rnd(*cache.k_pages.shape, dtype=dtype, seed=9))
        cache.v_pages.copy_(rnd(*cache.v_pages.shape, dtype=dtype, seed=10))
        qkv = rnd(ctx.n_tokens, (n_heads + 2 * n_kv) * D, dtype=dtype, seed=11)
        out = hip.paged_attention(qkv, n_heads, n_kv, D, 1 / math.sqrt(D), window, ctx, cache)
        ref = twin.paged_attention(qkv, n_heads, n_kv, D, 1 / math.sqrt(D), window, ctx, cache)
        torch.testing.assert_close(out.float(), ref.float(), **tol(dtype))
        hip.use_mfma_attention = False
        try:
            plain_kernel = hip.paged_attention(qkv, n_heads, n_kv, D, 1 / math.sqrt(D), window, ctx, cache)
        finally:
            hip.use_mfma_attention = True
        torch.testing.assert_close(plain_kernel.float(), ref.float(), **tol(dtype))


@pytest.mark.parametrize("geom", [(24, 8, 128, 16, None), (6, 2, 48, 16, 700), (32, 8, 64, 64, None)])
def test_decode_attention_of_a_sequence_does_not_depend_on_its_batch(hip, geom):
    """How a sequence's keys are split between workgroups and merged follows from its own length: alone, beside
    others, beside many, and under a larger bound on the length (as replayed graphs have it) its result is the
    same bit for bit.  Lengths on both sides of every number of splits (1, 2, 4, 8, 16 from 512 keys a split)."""
    n_heads, n_kv, D, ps, window = geom
    dtype = torch.bfloat16
    kv_lens = [1, 63, 511, 512, 1023, 1024, 1500, 2048, 2500, 4095, 4097, 9000]
    pages = sum(-(-kv // ps) for kv in kv_lens) + 5
    cache = Cache(pages, n_kv, ps, D, dtype, kv_lens, seed=8)
    cache.k_pages.copy_(rnd(*cache.k_pages.shape, dtype=dtype, seed=9))
    cache.v_pages.copy_(rnd(*cache.v_pages.shape, dtype=dtype, seed=10))
    qkv = rnd(len(kv_lens), (n_heads + 2 * n_kv) * D, dtype=dtype, seed=11)
    scale = 1 / math.sqrt(D)

    def run(which, bound=0, repeat=1):
        """Attention of the sequences ``which`` (each ``repeat`` times in the batch) as one decode step."""
        ids = [i for i in which for _ in range(repeat)]
        ctx = Ctx([1] * len(ids), [kv_lens[i] for i in ids])
        ctx.kv_bound = bound
        sub = Cache.__new__(Cache)
        sub.page_size, sub.k_pages, sub.v_pages = ps, cache.k_pages, cache.v_pages
        sub.block_table = cache.block_table[ids].contiguous()
        out = hip.paged_attention(qkv[ids].contiguous(), n_heads, n_kv, D, scale, window, ctx, sub)
        return {i: out[j * repeat] for j, i in enumerate(which)}

    everyone = list(range(len(kv_lens)))
    together = run(everyone)
    ref = twin.paged_attention(qkv, n_heads, n_kv, D, scale, window, Ctx([1] * len(kv_lens), kv_lens), cache)
    torch.testing.assert_close(torch.stack([together[i] for i in everyone]).float(), ref.float(), **tol(dtype))
    bounded = run(everyone, bound=16384)
    many = run(everyone, repeat=6)                    # 72 sequences: more workgroups than compute units
    # so many that one workgroup takes all the splits of a (sequence, kv head) in turn and merges them itself
    crowd = run(everyone, repeat=-(-600 // (n_kv * len(everyone))))
    crowd_bounded = run(everyone, bound=16384, repeat=-(-600 // (n_kv * len(everyone))))
    for i in everyone:
        alone = run([i])[i]
        assert torch.equal(alone, together[i]), kv_lens[i]
        assert torch.equal(alone, bounded[i]), kv_lens[i]
        assert torch.equal(alone, many[i]), kv_lens[i]
        assert torch.equal(alone, crowd[i]), kv_lens[i]
        assert torch.equal(alone, crowd_bounded[i]), kv_lens[i]
    pair = run([3, 9])
    assert torch.equal(pair[3], together[3]) and torch.equal(pair[9], together[9])


def test_few_row_products_do_not_depend_on_the_number_of_rows(hip):
    """Up to 16 rows every product (plain, gated, into the residual, with the norm's row scale, with rotation and
    cache write) sums k in an order that K alone fixes: a row's result is the same bit for bit whether it runs
    alone, among 4, among 5 (another kernel shape from 5 rows on) or among 16."""
    from simple_inference_amd.kernels import ScaledRows
    dtype = torch.bfloat16
    for N, K in ((3072, 8192), (5120, 3072), (16384, 3072), (1008, 1024), (48, 192)):
        x, w = rnd(16, K, dtype=dtype, seed=1), rnd(N, K, dtype=dtype, seed=2, scale=K ** -0.5)
        full = hip.linear(x, w)
        full32 = hip.linear(x, w, out_float32=True)
        for m in (1, 4, 5, 11):
            assert torch.equal(hip.linear(x[:m].contiguous(), w), full[:m]), (N, K, m)
            assert torch.equal(hip.linear(x[:m].contiguous(), w, out_float32=True), full32[:m]), (N, K, m)
            assert torch.equal(hip.linear(x[m - 1:m].contiguous(), w), full[m - 1:m]), (N, K, m)
    for inter, K in ((8192, 3072), (96, 320), (5120, 1024)):
        x = rnd(16, K, dtype=dtype, seed=3)
        w = rnd(2 * inter, K, dtype=dtype, seed=4, scale=K ** -0.5)
        full = hip.gated_linear(x, w)
        for m in (1, 4, 5, 11):
            assert torch.equal(hip.gated_linear(x[:m].contiguous(), w), full[:m]), (inter, K, m)
    # into the residual, and out of it again through the row scale of the products that follow
    hidden, inner, inter = 3072, 8192, 8192
    x = rnd(16, inner, dtype=dtype, seed=5)
    w = rnd(hidden, inner, dtype=dtype, seed=6, scale=inner ** -0.5)
    w_gu = rnd(2 * inter, hidden, dtype=dtype, seed=7, scale=hidden ** -0.5)
    res = rnd(16, hidden, seed=8, scale=2.0)
    gain = (rnd(hidden, seed=9, scale=0.3) + 1.0).contiguous()

    def through(m):
        r = res[:m].clone()
        scaled = hip.linear_into_residual(hip.pending_linear(x[:m].contiguous(), w), r, gain, 1e-5)
        assert isinstance(scaled, ScaledRows)
        return r, scaled.rows, hip.gated_linear(scaled, w_gu), hip.linear(scaled, w_gu)
    full = through(16)
    for m in (1, 4, 5, 11):
        for got, want in zip(through(m), full):
            assert torch.equal(got, want[:m]), m


@pytest.mark.parametrize("N, K", [(3072, 3072), (3070, 8192), (2048, 2048), (4099, 192)])
def test_a_tiled_copy_of_a_weight_changes_no_bit_of_the_product_into_the_residual(hip, N, K):
    """The product into the residual reads, where the kernels made one, a copy of the weight laid out in the order
    of its loads.  The same elements meet in the same sums: residual, scaled rows and sums of squares are the same
    bit for bit as from the weight as it is, for every number of rows, also where the last block of rows is short
    (3,070 and 4,099 rows).  A weight changed in place after the copy was made is read as it is."""
    dtype = torch.bfloat16
    x = rnd(16, K, dtype=dtype, seed=1)
    w = rnd(N, K, dtype=dtype, seed=2, scale=K ** -0.5)
    res = rnd(16, N, seed=3, scale=2.0)
    gain = (rnd(N, seed=4, scale=0.3) + 1.0).contiguous()

    def through(m):
        r = res[:m].clone()
        scaled = hip.linear_into_residual(hip.pending_linear(x[:m].contiguous(), w), r, gain, 1e-5)
        return r, scaled.rows, scaled.partials[:, :m].clone()

    plain = {m: through(m) for m in (1, 7, 16)}
    made = hip.prepare_pending_weight(w)
    assert made == (hip.core.sia_gemm_skinny_tile_height(N) > 0)
    for m, want in plain.items():
        for got, expected in zip(through(m), want):
            assert torch.equal(got, expected), (N, K, m)
    if made:
        assert hip._tiled_copy(w) is not None
        w.mul_(2.0)                                    # the copy no longer says what the weight holds
        assert hip._tiled_copy(w) is None
        r, rows, _ = through(5)
        want = res[:5] + (x[:5].float() @ w.float().T).to(dtype).float()
        torch.testing.assert_close(r, want, atol=2e-2, rtol=2e-2)
        assert hip.prepare_pending_weight(w) and hip._tiled_copy(w) is not None
        for got, expected in zip(through(5), (r, rows)):
            assert torch.equal(got, expected)


@pytest.mark.parametrize("q_len, kv_len, window", [(130, 130, None), (900, 1000, None), (1900, 1900, None),
                                                  (1900, 2100, 300)])
def test_matrix_core_prefill_in_each_workgroup_shape(hip, q_len, kv_len, window):
    """The prefill kernel picks one of three workgroup shapes by the number of workgroups: with 34 heads, 130
    tokens take the split shape (64 tokens, even and odd key tiles on two sets of waves, merged at the end),
    900 the 8-wave shape and 1,900 the wide one.  Lengths are no multiples of a tile."""
    n_heads, n_kv, D, ps = 34, 2, 16, 16
    dtype = torch.bfloat16
    ctx = Ctx([q_len, 3], [kv_len, 40])
    cache = Cache(-(-kv_len // ps) + 8, n_kv, ps, D, dtype, [kv_len, 40], seed=31)
    cache.k_pages.copy_(rnd(*cache.k_pages.shape, dtype=dtype, seed=32))
    cache.v_pages.copy_(rnd(*cache.v_pages.shape, dtype=dtype, seed=33))
    qkv = rnd(ctx.n_tokens, (n_heads + 2 * n_kv) * D, dtype=dtype, seed=34, scale=2.0)
    out = hip.paged_attention(qkv, n_heads, n_kv, D, 1 / math.sqrt(D), window, ctx, cache)
    ref = twin.paged_attention(qkv, n_heads, n_kv, D, 1 / math.sqrt(D), window, ctx, cache)
    torch.testing.assert_close(out.float(), ref.float(), **tol(dtype))


def test_matrix_core_prefill_in_workgroups_of_256_tokens(hip):
    """Very many workgroups (128 heads, 2,500 tokens) take the shape of 8 waves of 32 tokens; a second and a third
    run in the same launch, shorter than a workgroup and a little longer than one, and a window."""
    n_heads, n_kv, D, ps = 128, 8, 16, 16
    dtype = torch.bfloat16
    q_lens, kv_lens = [2500, 40, 300], [2700, 40, 555]
    ctx = Ctx(q_lens, kv_lens)
    cache = Cache(sum(-(-kv // ps) for kv in kv_lens) + 8, n_kv, ps, D, dtype, kv_lens, seed=41)
    cache.k_pages.copy_(rnd(*cache.k_pages.shape, dtype=dtype, seed=42))
    cache.v_pages.copy_(rnd(*cache.v_pages.shape, dtype=dtype, seed=43))
    qkv = rnd(ctx.n_tokens, (n_heads + 2 * n_kv) * D, dtype=dtype, seed=44, scale=2.0)
    lib = hip._attn_lib(D)
    assert lib.sia_attn_prefill_rows_long() == 256
    assert sum(-(-q // lib.sia_attn_prefill_rows()) for q in q_lens) * n_heads >= 2400   # the launch takes that shape
    for window in (None, 700):
        out = hip.paged_attention(qkv, n_heads, n_kv, D, 1 / math.sqrt(D), window, ctx, cache)
        ref = twin.paged_attention(qkv, n_heads, n_kv, D, 1 / math.sqrt(D), window, ctx, cache)
        torch.testing.assert_close(out.float(), ref.float(), **tol(dtype))


def test_matrix_core_attention_runs_longer_than_a_block_table_window(hip, monkeypatch):
    """A wave holds 64 block-table entries at a time.  With pages of 64, runs of more than 4,096 keys that
    start in the middle of a page (tiles are 32 keys) must reload the entries at a page's edge: one decoded
    token over 17,500 keys (four runs of about 4,380 keys), and a prompt portion under a window of 5,000."""
    n_heads, n_kv, D, ps = 2, 1, 16, 64
    dtype = torch.bfloat16
    # one workgroup per (sequence, kv head), whatever the length: a wave's run of keys is then longer than a window
    monkeypatch.setattr(hip._attn_lib(D), "sia_attn_decode_max_splits", lambda kv_bound, window: 1)
    for q_lens, kv_lens, window in (([1], [17500], None), ([1], [17500], 9001), ([70], [9000], 5000)):
        ctx = Ctx(q_lens, kv_lens)
        cache = Cache(-(-kv_lens[0] // ps) + 3, n_kv, ps, D, dtype, kv_lens, seed=21)
        cache.k_pages.copy_(rnd(*cache.k_pages.shape, dtype=dtype, seed=22))
        cache.v_pages.copy_(rnd(*cache.v_pages.shape, dtype=dtype, seed=23))
        qkv = rnd(ctx.n_tokens, (n_heads + 2 * n_kv) * D, dtype=dtype, seed=24, scale=3.0)
        out = hip.paged_attention(qkv, n_heads, n_kv, D, 1 / math.sqrt(D), window, ctx, cache)
        ref = twin.paged_attention(qkv, n_heads, n_kv, D, 1 / math.sqrt(D), window, ctx, cache)
        torch.testing.assert_close(out.float(), ref.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("q_len", [1, 40])
def test_attention_finds_one_key_at_every_kind_of_edge(hip, dtype, q_len):
    """One key among hundreds is made to stand out; the output must be its value row.  The key is put at
    the edges where an indexing fault would lose it: first and last offset of a page, of a 32- and
    64-key tile, the first key, the newest key, and both sides of a window's edge.  (700 keys are 22 tiles, which
    the decode kernel does not split; longer sequences and their splits have a test of their own below.)"""
    n_heads, n_kv, D, ps = 4, 2, 64, 16
    kv = 700
    ctx = Ctx([q_len], [kv])
    last = kv - 1                       # the position of the last query
    direction = torch.nn.functional.normalize(rnd(D, seed=3), dim=0)
    base_k = 0.01 * rnd(64, n_kv, ps, D, seed=1)
    values = rnd(64, n_kv, D, ps, seed=2)
    qkv = torch.zeros(q_len, (n_heads + 2 * n_kv) * D)
    qkv[:, :n_heads * D] = (30.0 * direction).repeat(n_heads)
    qkv = qkv.to(dtype).to(DEV)
    cache = Cache(64, n_kv, ps, D, dtype, [kv])
    cache.v_pages.copy_(values.to(dtype))
    window = 300
    edge = last - window + 1            # oldest key the last query sees through the window
    for far, win, seen in [(0, None, True), (15, None, True), (16, None, True), (31, None, True), (32, None, True),
                           (63, None, True), (64, None, True), (255, None, True), (256, None, True),
                           (511, None, True), (512, None, True), (last - q_len, None, True), (last, None, True),
                           (edge, window, True), (edge - 1, window, False), (edge + 1, window, True)]:
        cache.k_pages.copy_(base_k.to(dtype))
        page = int(cache.block_table[0, far // ps])
        cache.k_pages[page, :, far % ps] = (30.0 * direction).to(dtype)
        out = hip.paged_attention(qkv, n_heads, n_kv, D, 1 / math.sqrt(D), win, ctx, cache).float()
        row = out[-1].view(n_heads, D)      # the last query sees every key up to ``last``
        for h in range(n_heads):
            want = cache.v_pages[page, h // 2, :, far % ps].float()
            close = torch.allclose(row[h], want, rtol=2e-2, atol=2e-2)
            assert close == seen, (far, win, h)


def _decode_splits(n_tiles):
    """How many workgroups share a sequence of that many visible key tiles (the kernel's own rule, written down a
    second time so that the test knows where the runs of tiles begin)."""
    s = 1
    while s < 32 and 2 * s * 16 <= n_tiles:
        s *= 2
    return s


@pytest.mark.parametrize("kv, window", [(1100, None), (2500, None), (9000, None), (9000, 5000)])
def test_decode_attention_finds_one_far_key_however_its_runs_are_spread(hip, kv, window):
    """A decoding sequence of 1,100 to 9,000 keys is cut into 2 to 16 splits of four runs of tiles each, and the
    runs are spread over workgroups in three ways: a workgroup a run (few sequences), a workgroup a split (some),
    one workgroup for all of a sequence's runs (a crowd).  One key is made to stand out and the output must be its
    value row, with the key at the first and the last position of runs in the middle of a split, at a split's
    edge, in the very first and the very last run, and on either side of a window's edge; in each of the three ways,
    and in a grid sized for a longer sequence than the step holds."""
    n_heads, n_kv, D, ps = 4, 2, 64, 16
    dtype = torch.bfloat16
    lib = hip._attn_lib(D)
    last = kv - 1
    lo_all = max(0, last - window + 1) if window else 0
    t_first, n_tiles = lo_all // 32, last // 32 - lo_all // 32 + 1
    n_splits = _decode_splits(n_tiles)
    n_runs = 4 * n_splits
    assert n_splits >= 2
    begin = lambda run: (t_first + run * n_tiles // n_runs) * 32         # first key of a run
    runs = sorted({1, 2, 4, 5, n_runs // 2, n_runs - 4, n_runs - 1})
    places = {max(lo_all, begin(run)) for run in runs} | {begin(run) - 1 for run in runs if begin(run) - 1 >= lo_all}
    cases = [(p, True) for p in sorted(places | {lo_all, last})]
    if window:
        cases += [(lo_all - 1, False), (lo_all + 1, True)]
    n_pages = -(-kv // ps)
    direction = torch.nn.functional.normalize(rnd(D, seed=3), dim=0)
    base_k = (0.01 * rnd(n_pages, n_kv, ps, D, seed=1)).to(dtype)
    cache = Cache(n_pages, n_kv, ps, D, dtype, [kv], seed=5)
    cache.v_pages.copy_(rnd(n_pages, n_kv, D, ps, seed=2).to(dtype))
    row = cache.block_table[0].clone()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    crowd = -(-cus // n_kv) + 3                                            # a (sequence, kv head) pair a compute unit
    some = -(-cus // (n_kv * n_splits)) + 1                                # more splits than compute units
    seen_modes = set()
    for n_seqs, bound, want_mode in ((1, 0, 2), (some, 0, 0), (crowd, 0, 1), (1, 4 * kv, 2), (crowd, 2 * kv, 1)):
        ctx = Ctx([1] * n_seqs, [kv] * n_seqs)
        ctx.kv_bound = bound
        max_splits = lib.sia_attn_decode_max_splits(bound or kv, window or 0)
        if some * n_kv >= cus and want_mode == 0:
            continue                                                       # two splits only: no step takes that way
        assert lib.sia_attn_decode_mode(n_seqs, n_heads, n_kv, max_splits) == want_mode, (n_seqs, bound)
        seen_modes.add(want_mode)
        cache.block_table = row.repeat(n_seqs, 1).contiguous()             # every sequence reads the same pages
        qkv = torch.zeros(n_seqs, (n_heads + 2 * n_kv) * D)
        qkv[:, :n_heads * D] = (30.0 * direction).repeat(n_heads)
        qkv = qkv.to(dtype).to(DEV)
        for far, seen in cases:
            cache.k_pages.copy_(base_k)
            page = int(row[far // ps])
            cache.k_pages[page, :, far % ps] = (30.0 * direction).to(dtype)
            out = hip.paged_attention(qkv, n_heads, n_kv, D, 1 / math.sqrt(D), window, ctx, cache).float()
            for s in sorted({0, n_seqs // 2, n_seqs - 1}):
                got = out[s].view(n_heads, D)
                for h in range(n_heads):
                    want = cache.v_pages[page, h // 2, :, far % ps].float()
                    assert torch.allclose(got[h], want, rtol=2e-2, atol=2e-2) == seen, (n_seqs, bound, far, s, h)
    assert {1, 2} <= seen_modes


@pytest.mark.parametrize("vocab", [16, 1000, 128256])
def test_sample_matches_twin(hip, vocab):
    rows = 12
    logits = rnd(rows, vocab, seed=1, scale=2.0)
    temperature = torch.tensor([0, 0, 1, 1, 0.7, 0.7, 1.3, 1, 1, 0.5, 1, 2], dtype=torch.float32, device=DEV)
    top_k = torch.tensor([0, 5, 0, 0, 5, 0, 50, 1, 0, 3, vocab, 7], dtype=torch.int32, device=DEV)
    top_p = torch.tensor([1, 1, 1, 1, 1, 0.9, 0.5, 1, 0.0, 0.8, 1, 0.3], dtype=torch.float32, device=DEV)
    for seed in range(4):
        u = torch.rand(rows, generator=torch.Generator().manual_seed(seed)).to(DEV)
        got = hip.sample(logits, temperature, top_k, top_p, u)
        ref = twin.sample(logits, temperature, top_k, top_p, u)
        assert got.tolist() == ref.tolist(), (seed, got.tolist(), ref.tolist())


@pytest.mark.parametrize("vocab", [7, 331, 50257])
def test_sample_filters_at_their_edges(hip, vocab):
    """Rows made so that a filter's edge shows: equal values (kept or dropped together), a k that is one short
    of everything, a p so small that only the top stays, a single dominant token, values of both signs far
    apart, and draws at both ends of the unit interval.  The hints of which filters exist must not matter."""
    g = torch.Generator().manual_seed(vocab)
    rows = []
    flat = torch.zeros(vocab)                                        # all equal
    steps = torch.arange(vocab, dtype=torch.float32).flip(0) * 0.25   # strictly falling
    pairs = (torch.arange(vocab) // 2).float().flip(0) * 0.5          # equal pairs
    spike = torch.randn(vocab, generator=g); spike[vocab // 3] = 30.0
    wide = torch.randn(vocab, generator=g) * 40.0
    shuffled = steps[torch.randperm(vocab, generator=g)]
    cases = []
    for base in (flat, steps, pairs, spike, wide, shuffled):
        ties = base is flat or base is pairs   # a sort splits equal values as it likes: no top-p oracle for them
        for k, p in ((0, 1.0), (1, 1.0), (3, 1.0), (vocab - 1, 1.0), (0, 1e-6), (0, 0.5), (4, 0.7), (0, 0.999)):
            if not (ties and p < 1.0):
                cases.append((base, 0.8, k, p))
    logits = torch.stack([c[0] for c in cases]).to(DEV)
    temperature = torch.tensor([c[1] for c in cases], dtype=torch.float32, device=DEV)
    top_k = torch.tensor([c[2] for c in cases], dtype=torch.int32, device=DEV)
    top_p = torch.tensor([c[3] for c in cases], dtype=torch.float32, device=DEV)
    for u_value in (1e-6, 0.37, 0.999999):
        u = torch.full((len(cases),), u_value, dtype=torch.float32, device=DEV)
        got = hip.sample(logits, temperature, top_k, top_p, u)
        ref = twin.sample(logits, temperature, top_k, top_p, u)
        assert got.tolist() == ref.tolist(), (u_value, [i for i, (a, b) in enumerate(zip(got.tolist(), ref.tolist())) if a != b])
    # equal values are kept or dropped together: under any top-p, all of a row of equal values can be drawn
    n = 5
    flat_rows = flat.repeat(n, 1).to(DEV)
    u = torch.linspace(0.01, 0.99, n, device=DEV)
    got = hip.sample(flat_rows, torch.full((n,), 0.8, device=DEV), torch.zeros(n, dtype=torch.int32, device=DEV),
                     torch.full((n,), 0.3, device=DEV), u)
    assert got.tolist() == [min(vocab - 1, int(x * vocab)) for x in u.tolist()]
    # rows without a filter, sampled with the hint that there is none
    plain_rows = [i for i, c in enumerate(cases) if c[2] == 0 and c[3] == 1.0]
    sel = torch.tensor(plain_rows, device=DEV)
    u = torch.full((len(plain_rows),), 0.61, dtype=torch.float32, device=DEV)
    args = (logits[sel].contiguous(), temperature[sel].contiguous(), top_k[sel].contiguous(), top_p[sel].contiguous(), u)
    assert hip.sample(*args, filters=0).tolist() == hip.sample(*args).tolist() == twin.sample(*args).tolist()


def test_sample_does_not_care_what_its_workspace_held(hip):
    """The sampler sets to zero what it needs at zero: a workspace full of ones gives the tokens of a zeroed one,
    and the kernels object's own workspace, used by every call before this one, gives them too."""
    rows, vocab = 6, 3001
    logits = rnd(rows, vocab, seed=8, scale=2.5)
    temperature = torch.tensor([0.9, 0.0, 1.1, 0.6, 1.0, 0.8], dtype=torch.float32, device=DEV)
    top_k = torch.tensor([40, 0, 0, 7, 0, 2999], dtype=torch.int32, device=DEV)
    top_p = torch.tensor([0.9, 1.0, 0.6, 1.0, 1.0, 0.95], dtype=torch.float32, device=DEV)
    u = torch.tensor([0.11, 0.5, 0.93, 0.42, 0.77, 0.3], dtype=torch.float32, device=DEV)
    want = hip.sample(logits, temperature, top_k, top_p, u).tolist()
    assert want == twin.sample(logits, temperature, top_k, top_p, u).tolist()
    size = hip.core.sia_sample_workspace_bytes(rows)
    for fill in (0, 255, 1):
        out = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        workspace = torch.full((size,), fill, dtype=torch.uint8, device=DEV)
        code = hip.core.sia_sample(logits.data_ptr(), temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(),
                                   u.data_ptr(), out.data_ptr(), workspace.data_ptr(), rows, vocab, 7,
                                   torch.cuda.current_stream().cuda_stream)
        assert code == 0
        assert out.tolist() == want, fill


@pytest.mark.parametrize("vocab", [5, 1001, 4096, 128256])
def test_argmax_of_all_greedy_steps(hip, vocab):
    rows = 9
    logits = rnd(rows, vocab, seed=3, scale=3.0)
    logits[1] = 0.0                                   # all equal: index 0
    logits[2, vocab - 1] = 50.0                       # the last element
    logits[3, [vocab // 2, vocab - 2 if vocab > 2 else 0]] = 60.0   # a tie across chunks: the lower index
    z = lambda dt, v: torch.full((rows,), v, dtype=dt, device=DEV)
    args = (logits, z(torch.float32, 0.0), z(torch.int32, 0), z(torch.float32, 1.0), z(torch.float32, 0.5))
    spread = hip.sample(*args, all_greedy=True)
    assert spread.tolist() == hip.sample(*args).tolist()
    library = torch.argmax(logits, -1).tolist()
    assert [t for i, t in enumerate(spread.tolist()) if i not in (1, 3)] == [t for i, t in enumerate(library) if i not in (1, 3)]
    assert spread[1].item() == 0 and spread[2].item() == vocab - 1
    assert spread[3].item() == min(vocab // 2, vocab - 2 if vocab > 2 else 0)


def test_sample_greedy_is_argmax_with_lowest_index_on_ties(hip):
    logits = torch.zeros(3, 5000, device=DEV)
    logits[0, 4321] = 1.0
    logits[1, [17, 4000]] = 2.0
    z = lambda dt, v: torch.full((3,), v, dtype=dt, device=DEV)
    got = hip.sample(logits, z(torch.float32, 0.0), z(torch.int32, 0), z(torch.float32, 1.0), z(torch.float32, 0.5))
    assert got.tolist() == [4321, 17, 0]
