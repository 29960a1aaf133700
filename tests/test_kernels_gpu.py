"""Each HIP kernel alone against a plain float64/float32 torch formula of the same
operation, at sizes other than the tiny engines' (odd widths, many heads, long rows)."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def _tol(dtype):
    # float32 kernels: a few ulp of accumulated 32-bit rounding; bfloat16: one bf16 rounding
    # of the result (2^-8 relative) plus accumulated input rounding.
    return dict(rtol=2e-5, atol=2e-6) if dtype == torch.float32 else dict(rtol=1.6e-2, atol=2e-3)


@pytest.fixture(scope="module")
def ops():
    from torchlet_amd.kernels import ops
    return ops


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("V,H,T", [(300, 96, 7), (1031, 3584, 33)])
def test_embedding(ops, dtype, V, H, T):
    g = torch.Generator().manual_seed(0)
    table = torch.randn(V, H, generator=g).to(dtype).cuda()
    ids = torch.randint(0, V, (T,), generator=g, dtype=torch.int32).cuda()
    out = torch.empty(T, H, dtype=torch.float32, device="cuda")
    ops.embedding(ids, table, out)
    assert torch.equal(out, table.float()[ids.long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("wdtype", DTYPES)
@pytest.mark.parametrize("T,H,eps", [(5, 96, 1e-5), (19, 1000, 1e-6), (3, 5120, 1e-6), (2, 1001, 1e-6), (8, 3584, 1e-6), (2, 10000, 1e-5), (1, 20000, 1e-6)])
def test_add_rmsnorm(ops, dtype, wdtype, T, H, eps):
    if dtype == torch.float32 and wdtype == torch.bfloat16:
        pytest.skip("a 32-bit engine widens its vectors")
    g = torch.Generator().manual_seed(1)
    res = (torch.randn(T, H, generator=g) * 3).cuda()
    pend = torch.randn(T, H, generator=g).to(dtype).cuda()
    w = (1 + 0.1 * torch.randn(H, generator=g)).to(wdtype).cuda()
    ref_r = res.double() + pend.double()
    ref = ref_r * torch.rsqrt(ref_r.pow(2).mean(-1, keepdim=True) + eps) * w.double()
    # with pending: residual updated
    r1 = res.clone()
    out = torch.empty(T, H, dtype=dtype, device="cuda")
    ops.add_rmsnorm(r1, pend, w, eps, out)
    torch.testing.assert_close(r1.double(), ref_r, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(out.double(), ref, **_tol(dtype))
    # without pending: residual untouched
    r2 = res.clone()
    ops.add_rmsnorm(r2, None, w, eps, out)
    assert torch.equal(r2, res)
    ref2 = res.double() * torch.rsqrt(res.double().pow(2).mean(-1, keepdim=True) + eps) * w.double()
    torch.testing.assert_close(out.double(), ref2, **_tol(dtype))
    # selected rows: nothing written back
    rows = torch.tensor([T - 1, 0, T - 1], dtype=torch.int32, device="cuda")
    r3 = res.clone()
    out3 = torch.empty(3, H, dtype=dtype, device="cuda")
    ops.add_rmsnorm(r3, pend, w, eps, out3, rows)
    assert torch.equal(r3, res)
    torch.testing.assert_close(out3.double(), ref[rows.long()], **_tol(dtype))


@pytest.mark.parametrize("M", [1, 8, 16, 33, 64, 65, 200, 513])
@pytest.mark.parametrize("N,K", [(3584, 18944), (100, 8192 + 200), (64, 64), (130, 4096)])
def test_linear_partials_and_their_sum_in_the_norm(ops, M, N, K):
    """Split-K slabs of partial sums: their sum is the product, and add_rmsnorm adds them up."""
    g = torch.Generator().manual_seed(M + N)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16).cuda()
    if M > 64 and K % 64:
        assert not ops.linear_partials_pay(M, N, K)
        with pytest.raises(ops.KernelError, match="multiple of 64"):
            ops.linear_partials(x, w)
        return
    parts = ops.linear_partials(x, w)
    assert parts.dim() == 3 and parts.shape[1:] == (M, N) and parts.dtype == torch.float32
    assert 1 <= parts.shape[0] <= ops._lib("gemm").tl_gemm_partials_parts(M, N, K) <= 8      # as many slabs as the library said at most
    ref = x.double() @ w.double().T
    tol32 = dict(rtol=2e-5, atol=8 * 2 ** -24 * math.sqrt(K) * float(ref.pow(2).mean().sqrt()))
    torch.testing.assert_close(parts.double().sum(0), ref, **tol32)
    res = torch.randn(M, N, generator=g).cuda()
    wn = (1 + 0.1 * torch.randn(N, generator=g)).to(torch.bfloat16).cuda()
    r = res.clone()
    out = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    ops.add_rmsnorm(r, parts, wn, 1e-6, out)
    total = res.double() + ref
    torch.testing.assert_close(r.double(), total, rtol=1e-5, atol=2e-5)
    refn = total * torch.rsqrt(total.pow(2).mean(-1, keepdim=True) + 1e-6) * wn.double()
    torch.testing.assert_close(out.double(), refn, **_tol(torch.bfloat16))
    rows = torch.tensor([M - 1, 0], dtype=torch.int32, device="cuda")
    out2 = torch.empty(2, N, dtype=torch.bfloat16, device="cuda")
    r2 = res.clone()
    ops.add_rmsnorm(r2, parts, wn, 1e-6, out2, rows)
    assert torch.equal(r2, res)
    torch.testing.assert_close(out2.double(), refn[rows.long()], **_tol(torch.bfloat16))


def test_a_portion_of_2048_rows_against_a_narrow_down_projection_is_split_in_two(ops):
    """2048 rows against a 5120 x 27648 matrix: 160 tiles of 256 x 256 leave three compute units in eight idle, and
    128 tiles of 256 x 320 with K in two halves are one round of 256 work-groups.  The plan is that one, and its sum
    is the product."""
    M, N, K = 2048, 5120, 27648
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(M, K, generator=g, device="cuda").to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g, device="cuda") / math.sqrt(K)).to(torch.bfloat16)
    assert ops.linear_partials_pay(M, N, K)
    parts = ops.linear_partials(x, w)
    if ops.compute_units() == ops.MEASURED_COMPUTE_UNITS:
        assert parts.shape[0] == 2
    ref = x.double() @ w.double().T
    tol32 = dict(rtol=2e-5, atol=8 * 2 ** -24 * math.sqrt(K) * float(ref.pow(2).mean().sqrt()))
    torch.testing.assert_close(parts.double().sum(0), ref, **tol32)


def test_rmsnorm_zero_row_is_zero_not_nan(ops):
    res = torch.zeros(2, 64, device="cuda")
    w = torch.ones(64, device="cuda")
    out = torch.full((2, 64), 7.0, device="cuda")
    ops.add_rmsnorm(res, None, w, 1e-6, out)
    assert torch.equal(out, torch.zeros_like(out))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K,bias", [(1, 300, 96, True), (7, 129, 200, False), (65, 64, 17, True), (130, 513, 1000, True)])
def test_linear(ops, dtype, M, N, K, bias):
    g = torch.Generator().manual_seed(2)
    x = torch.randn(M, K, generator=g).to(dtype).cuda()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(dtype).cuda()
    b = torch.randn(N, generator=g).to(dtype).cuda() if bias else None
    ref = x.double() @ w.double().T + (b.double() if bias else 0)
    # A 32-bit sum of K products of size ~rms/sqrt(K) carries a rounding error of about
    # eps * sqrt(K) * rms (random walk); 8 of those bound the largest of ~1e5 elements.
    tol32 = dict(rtol=2e-5, atol=8 * 2 ** -24 * math.sqrt(K) * float(ref.pow(2).mean().sqrt()))
    out = torch.empty(M, N, dtype=dtype, device="cuda")
    ops.linear(x, w, b, out)
    torch.testing.assert_close(out.double(), ref, **(tol32 if dtype == torch.float32 else _tol(dtype)))
    out32 = torch.empty(M, N, dtype=torch.float32, device="cuda")
    ops.linear(x, w, b, out32)
    torch.testing.assert_close(out32.double(), ref, **tol32)
    # a strided input view (columns of a wider buffer)
    wide = torch.zeros(M, K + 24, dtype=dtype, device="cuda")
    wide[:, 8:8 + K] = x
    ops.linear(wide[:, 8:8 + K], w, b, out32)
    torch.testing.assert_close(out32.double(), ref, **tol32)


@pytest.mark.parametrize("M,N,K,bias", [(17, 129, 200, True), (65, 64, 20, False), (130, 513, 1000, True), (64, 300, 4, True),
                                        (300, 3584, 3584, False), (1000, 257, 1028, True), (33, 1, 8, True), (2048, 130, 3584, True)])
def test_linear_many_rows_in_32_bit_on_matrix_cores(ops, M, N, K, bias):
    """v_mfma_f32_32x32x2_f32: true 32-bit products and sums.  Against float64 with the bound of a 32-bit sum; the
    general v_fma_f32 kernel agrees with it to rounding; a row's result does not depend on how many rows there are
    beside it or where it lies (bitwise: its sum runs in one order); inputs whose products need every bit of a
    32-bit mantissa show that nothing is rounded to a shorter format on the way."""
    g = torch.Generator().manual_seed(M + N + K)
    x = torch.randn(M, K, generator=g).cuda()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).cuda()
    b = torch.randn(N, generator=g).cuda() if bias else None
    ref = x.double() @ w.double().T + (b.double() if bias else 0)
    tol32 = dict(rtol=2e-5, atol=8 * 2 ** -24 * math.sqrt(K) * float(ref.pow(2).mean().sqrt()))
    out = torch.full((M, N), float("nan"), device="cuda")
    ops.linear_f32_variant(x, w, b, out, True)
    torch.testing.assert_close(out.double(), ref, **tol32)
    fma = torch.empty(M, N, device="cuda")
    ops.linear_f32_variant(x, w, b, fma, False)
    torch.testing.assert_close(fma.double(), ref, **tol32)
    through = torch.empty(M, N, device="cuda")
    ops.linear(x, w, b, through)                               # the dispatch takes the matrix-core kernel from 17 rows on
    assert torch.equal(through, out)
    # some rows alone, elsewhere in a tile, inside a wider buffer: the same bits
    rows = [M - 1, 0, M // 2] * 7
    wide = torch.zeros(len(rows), K + 12, device="cuda")
    wide[:, 4:4 + K] = x[rows]
    few = torch.empty(len(rows), N, device="cuda")
    ops.linear_f32_variant(wide[:, 4:4 + K], w, b, few, True)
    assert torch.equal(few, out[rows])
    # operands 1 + d with d below 2^-12 and random signs: what tells them apart lies in the low bits of a 24-bit
    # mantissa.  A 32-bit sum of K such products (partial sums of size ~sqrt(K), each addition off by half an ulp of
    # that) stays within 4 * 2^-24 * K; operands cut to a shorter mantissa on the way would leave that bound far behind,
    # as the same product of bfloat16-rounded operands does.
    xe = (1 + torch.rand(M, K, generator=g) * 2 ** -12).cuda()
    we = ((1 + torch.rand(N, K, generator=g) * 2 ** -12) * (torch.randint(0, 2, (N, K), generator=g) * 2 - 1)).cuda()
    exact = xe.double() @ we.double().T
    got = torch.empty(M, N, device="cuda")
    ops.linear_f32_variant(xe, we, None, got, True)
    bound = 4 * 2 ** -24 * K
    assert float((got.double() - exact).abs().max()) < bound
    if M * N * K >= 1 << 16:
        cut = xe.bfloat16().double() @ we.bfloat16().double().T
        assert float((cut - exact).abs().max()) > 3 * bound


@pytest.mark.parametrize("M", [1, 2, 3, 7, 8, 13, 16])
@pytest.mark.parametrize("N,K", [(37, 100), (300, 1024), (129, 1028), (4608, 3584), (1, 2052), (64, 18944)])
def test_linear_few_rows_in_32_bit(ops, M, N, K):
    """The weight-streaming kernel of the 32-bit decode step: every count of rows, an odd number
    of weight rows, K of less than one, exactly one and several chunks with a tail; against a
    float64 product, and a row's result is the same whatever other rows stand beside it."""
    g = torch.Generator().manual_seed(M * 11 + N)
    x = torch.randn(M, K, generator=g).cuda()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).cuda()
    b = torch.randn(N, generator=g).cuda()
    ref = x.double() @ w.double().T + b.double()
    tol32 = dict(rtol=2e-5, atol=8 * 2 ** -24 * math.sqrt(K) * float(ref.pow(2).mean().sqrt()))
    out = torch.full((M, N), float("nan"), device="cuda")
    ops.linear(x, w, b, out)
    torch.testing.assert_close(out.double(), ref, **tol32)
    # two kernels serve these row counts (multiply-adds up to 8 rows, the matrix cores' true 32-bit instruction from 9
    # on): each agrees with float64, and in each a row's sum runs in one order whatever stands beside it (bitwise)
    for variant in (2, 3):
        got = torch.full((M, N), float("nan"), device="cuda")
        ops.linear_f32_variant(x, w, b, got, variant)
        torch.testing.assert_close(got.double(), ref, **tol32)
        alone = torch.empty(1, N, device="cuda")
        ops.linear_f32_variant(x[M - 1:], w, b, alone, variant)
        assert torch.equal(alone[0], got[M - 1]), f"variant {variant}"
        if variant == (3 if M > 8 else 2):
            assert torch.equal(got, out)                   # the dispatch's choice
    wide = torch.zeros(M, K + 24, device="cuda")          # a strided input view, a wider output
    wide[:, 8:8 + K] = x
    out2 = torch.full((M, N + 5), 3.0, device="cuda")
    ops.linear(wide[:, 8:8 + K], w, None, out2[:, :N])
    torch.testing.assert_close(out2[:, :N].double(), ref - b.double(), **tol32)
    assert bool((out2[:, N:] == 3.0).all())


@pytest.mark.parametrize("M", [1, 7, 16])
@pytest.mark.parametrize("N,K,blocks,rows", [(3584, 512, 1, 14), (4608, 320, 2, 18), (1000, 200, 1, 4), (1003, 128, 2, 31),
                                             (530, 264, 2, 17), (4099, 64, 1, 16), (700, 96, 1, 1)])
def test_linear_few_rows_in_strips_of_any_number_of_rows(ops, M, N, K, blocks, rows):
    """A matrix dealt to the compute units in equal shares: strips of a number of weight rows that is no
    multiple of 16, a last strip that is shorter still; every output written once, nothing beside them."""
    g = torch.Generator().manual_seed(M + N + rows)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16).cuda()
    b = torch.randn(N, generator=g).to(torch.bfloat16).cuda()
    ref = x.double() @ w.double().T + b.double()
    wide = torch.full((M + 1, N + 9), float("nan"), device="cuda")
    ops.linear_few_rows_variant(x, w, b, wide[:M, :N], blocks, 8, rows)
    tol32 = dict(rtol=2e-5, atol=8 * 2 ** -24 * math.sqrt(K) * float(ref.pow(2).mean().sqrt()))
    torch.testing.assert_close(wide[:M, :N].double(), ref, **tol32)
    assert bool(wide[:M, N:].isnan().all()) and bool(wide[M].isnan().all())
    plain = torch.empty(M, N, device="cuda")
    ops.linear_few_rows_variant(x, w, b, plain, blocks, 8, 0)
    assert torch.equal(plain, wide[:M, :N]), "the sums of a row do not depend on the strip it lies in"
    with pytest.raises(ops.KernelError, match="holds up to"):
        ops.linear_few_rows_variant(x, w, b, plain, blocks, 8, 16 * blocks + 1)


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M", [1, 5, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(48, 64), (129, 200), (4608, 3584), (3584, 1000), (16400, 256), (33000, 128)])
def test_linear_few_rows_on_matrix_cores(ops, out_dtype, M, N, K):
    """The weight-streaming kernel of the decode step: every choice of strips per wave and of
    waves along K, tails in M, N and K, against a float64 product of the same bfloat16 values."""
    g = torch.Generator().manual_seed(M * 7 + N)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16).cuda()
    b = torch.randn(N, generator=g).to(torch.bfloat16).cuda()
    ref = x.double() @ w.double().T + b.double()
    out = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
    ops.linear(x, w, b, out)
    # products of bfloat16 values are exact in 32-bit; only the sums round
    tol32 = dict(rtol=2e-5, atol=8 * 2 ** -24 * math.sqrt(K) * float(ref.pow(2).mean().sqrt()))
    torch.testing.assert_close(out.double(), ref, **(tol32 if out_dtype == torch.float32 else _tol(torch.bfloat16)))
    # the same through the general kernel: both are the engine's answer for some shape
    gen = torch.empty_like(out)
    ops.linear(x, w, b, gen, general=True)
    torch.testing.assert_close(out.double(), gen.double(), **(tol32 if out_dtype == torch.float32 else _tol(torch.bfloat16)))
    # a strided input view with aligned rows
    wide = torch.zeros(M, K + 40, dtype=torch.bfloat16, device="cuda")
    wide[:, 8:8 + K] = x
    out2 = torch.empty_like(out)
    ops.linear(wide[:, 8:8 + K], w, None, out2)
    torch.testing.assert_close(out2.double(), ref - b.double(), **(tol32 if out_dtype == torch.float32 else _tol(torch.bfloat16)))


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("tile", [(128, 128, 32), (128, 128, 64), (64, 128, 64), (256, 256, 64)])
@pytest.mark.parametrize("M,N,K", [(65, 129, 64), (300, 520, 200), (1000, 257, 1000), (2, 48, 3584)])
def test_linear_many_rows_on_matrix_cores(ops, out_dtype, tile, M, N, K):
    """Every tile shape of the shared-memory matrix-core kernel, with tails in M, N and K."""
    g = torch.Generator().manual_seed(M + N + K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16).cuda()
    b = torch.randn(N, generator=g).to(torch.bfloat16).cuda()
    ref = x.double() @ w.double().T + b.double()
    out = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
    ops.linear_many_rows_variant(x, w, b, out, *tile)
    tol32 = dict(rtol=2e-5, atol=8 * 2 ** -24 * math.sqrt(K) * float(ref.pow(2).mean().sqrt()))
    torch.testing.assert_close(out.double(), ref, **(tol32 if out_dtype == torch.float32 else _tol(torch.bfloat16)))
    wide = torch.zeros(M, K + 40, dtype=torch.bfloat16, device="cuda")
    wide[:, 16:16 + K] = x
    out2 = torch.empty_like(out)
    ops.linear_many_rows_variant(wide[:, 16:16 + K], w, None, out2, *tile)
    torch.testing.assert_close(out2.double(), ref - b.double(), **(tol32 if out_dtype == torch.float32 else _tol(torch.bfloat16)))


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("tile", [(64, 64), (64, 128), (64, 192), (64, 256), (64, 320), (128, 128), (128, 192), (128, 256), (256, 128), (192, 256), (256, 192), (256, 256), (256, 160)])
@pytest.mark.parametrize("M,N,K", [(65, 129, 64), (300, 520, 192), (1000, 257, 1024), (33, 48, 3584), (40, 4608, 128), (513, 700, 320)])
def test_linear_many_rows_fetched_straight_into_shared_memory(ops, out_dtype, tile, M, N, K):
    """Every tile shape of the direct-load matrix-core kernel, with tails in M and N, one slab to
    many (fewer slabs than pipeline stages too), a bias, a strided x."""
    g = torch.Generator().manual_seed(M + N + K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16).cuda()
    b = torch.randn(N, generator=g).to(torch.bfloat16).cuda()
    ref = x.double() @ w.double().T + b.double()
    out = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
    ops.linear_direct_variant(x, w, b, out, *tile)
    tol32 = dict(rtol=2e-5, atol=8 * 2 ** -24 * math.sqrt(K) * float(ref.pow(2).mean().sqrt()))
    torch.testing.assert_close(out.double(), ref, **(tol32 if out_dtype == torch.float32 else _tol(torch.bfloat16)))
    wide = torch.zeros(M, K + 40, dtype=torch.bfloat16, device="cuda")
    wide[:, 16:16 + K] = x
    out2 = torch.full((M, N + 8), 5.0, dtype=out_dtype, device="cuda")      # rows of a wider buffer
    ops.linear_direct_variant(wide[:, 16:16 + K], w, None, out2[:, :N], *tile)
    torch.testing.assert_close(out2[:, :N].double(), ref - b.double(), **(tol32 if out_dtype == torch.float32 else _tol(torch.bfloat16)))
    assert bool((out2[:, N:] == 5.0).all())


@pytest.mark.parametrize("M", [2048, 4096])
@pytest.mark.parametrize("N,K", [(5120, 1024), (7168, 640), (4608, 1088)])
def test_linear_of_thousands_of_rows_against_narrow_matrices_whatever_tile_it_picks(ops, M, N, K):
    """Whole prompt portions against matrices for which the planner weighs its widest tiles against each other (256 x 256,
    256 x 160, 192 x 256; one round of tiles or two): whichever it takes, the product is the product."""
    g = torch.Generator(device="cuda").manual_seed(M + N + K)
    x = torch.randn(M, K, generator=g, device="cuda").to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g, device="cuda") / math.sqrt(K)).to(torch.bfloat16)
    b = torch.randn(N, generator=g, device="cuda").to(torch.bfloat16)
    ref = x.double() @ w.double().T + b.double()
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    ops.linear(x, w, b, out)
    torch.testing.assert_close(out.double(), ref, **_tol(torch.bfloat16))
    parts = ops.linear_partials(x, w)
    tol32 = dict(rtol=2e-5, atol=8 * 2 ** -24 * math.sqrt(K) * float(ref.pow(2).mean().sqrt()))
    torch.testing.assert_close(parts.double().sum(0), ref - b.double(), **tol32)


def test_the_tile_product_refuses_rows_too_far_apart_for_its_32_bit_offsets(ops):
    """A lane of the direct-load kernel addresses its piece as a shared base plus a 32-bit offset from the tile's first
    row: rows of x that lie 2^23 elements apart put a tile's last row beyond that, and the launcher says so."""
    K, N = 64, 64
    store = torch.zeros(2 * (1 << 23), dtype=torch.bfloat16, device="cuda")
    x = store.view(2, 1 << 23)[:, :K]                       # two rows, 2^23 elements from one to the next
    w = torch.zeros(N, K, dtype=torch.bfloat16, device="cuda")
    out = torch.empty(2, N, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ops.KernelError, match="too long"):
        ops.linear_direct_variant(x, w, None, out, 256, 256)
    ops.linear_direct_variant(x, w, None, out, 64, 64)      # a tile of 64 rows reaches a quarter as far
    assert bool((out == 0).all())


@pytest.mark.parametrize("tile", [(64, 64, 0), (64, 192, 0), (64, 320, 0), (128, 192, 0), (128, 128, 0), (128, 128, 4), (128, 256, 0), (256, 128, 0), (192, 256, 0), (256, 192, 0), (256, 256, 0), (256, 320, 0), (256, 160, 0)])
@pytest.mark.parametrize("M,N,K,parts", [(65, 129, 128, 2), (128, 520, 1024, 4), (100, 3584, 2048, 8), (300, 257, 1088, 3), (7, 48, 3584, 7)])
def test_linear_split_over_k_on_every_tile_shape(ops, tile, M, N, K, parts):
    """Slabs of partial sums from every tile shape of the direct-load kernel (the four-slab 128 x 128
    instance among them), with tails in M and N and parts of unequal length: their sum is the product."""
    g = torch.Generator().manual_seed(M + N + K + parts)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16).cuda()
    ref = x.double() @ w.double().T
    slabs = ops.linear_direct_split_variant(x, w, tile[0], tile[1], parts, tile[2])
    assert slabs.shape == (parts, M, N)
    tol32 = dict(rtol=2e-5, atol=8 * 2 ** -24 * math.sqrt(K) * float(ref.pow(2).mean().sqrt()))
    torch.testing.assert_close(slabs.double().sum(0), ref, **tol32)
    k_per = -(-(K // 64) // parts) * 64
    torch.testing.assert_close(slabs[0].double(), x[:, :k_per].double() @ w[:, :k_per].double().T, **tol32)


@pytest.mark.parametrize("M", [1, 8, 16, 17, 32, 33, 64, 65, 300])
@pytest.mark.parametrize("I,K", [(128, 64), (200, 96), (112, 80), (18944, 256), (32768 + 40, 64), (100, 128), (36, 64)])
def test_linear_swiglu_fused(ops, M, I, K):
    """The gate/up product with the gate applied to the accumulators: every kernel behind it
    (few rows, 64-row tile, 128 and 256-row tiles), with I not a multiple of 32 or of 8."""
    g = torch.Generator().manual_seed(M + I)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
    gate = (torch.randn(I, K, generator=g) / math.sqrt(K) * 2).to(torch.bfloat16).cuda()
    up = (torch.randn(I, K, generator=g) / math.sqrt(K) * 2).to(torch.bfloat16).cuda()
    w = ops.interleave_gate_up(gate, up)
    assert w.shape == (-(-I // 32) * 64, K)
    out = torch.full((M, I + 8), float("nan"), dtype=torch.bfloat16, device="cuda")
    ops.linear_swiglu(x, w, out[:, :I])
    ref = torch.nn.functional.silu(x.double() @ gate.double().T) * (x.double() @ up.double().T)
    torch.testing.assert_close(out[:, :I].double(), ref, **_tol(torch.bfloat16))
    assert bool(out[:, I:].isnan().all())          # nothing is written beyond the I columns


@pytest.mark.parametrize("tile", [(64, 128), (64, 192), (64, 256), (128, 128), (128, 192), (128, 256), (256, 128), (192, 256), (256, 256)])
@pytest.mark.parametrize("M,I,K", [(17, 200, 64), (64, 18944, 128), (100, 1000, 320), (300, 36, 192)])
def test_linear_swiglu_fused_on_every_tile_shape(ops, tile, M, I, K):
    """The fused gate/up product on each tile shape by name (the dispatch picks by shape, and so would leave
    shapes untested that only large matrices get), tails in M and I, one slab to five."""
    g = torch.Generator().manual_seed(M + I)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
    gate = (torch.randn(I, K, generator=g) / math.sqrt(K) * 2).to(torch.bfloat16).cuda()
    up = (torch.randn(I, K, generator=g) / math.sqrt(K) * 2).to(torch.bfloat16).cuda()
    out = torch.full((M + 1, I + 8), float("nan"), dtype=torch.bfloat16, device="cuda")
    ops.linear_swiglu_direct_variant(x, ops.interleave_gate_up(gate, up), out[:M, :I], *tile)
    ref = torch.nn.functional.silu(x.double() @ gate.double().T) * (x.double() @ up.double().T)
    torch.testing.assert_close(out[:M, :I].double(), ref, **_tol(torch.bfloat16))
    assert bool(out[:M, I:].isnan().all()) and bool(out[M].isnan().all())


def _rope_ref(x, pos, theta):
    """x [T, heads, hd] float64; split-half pairing."""
    hd = x.shape[-1]
    j = torch.arange(0, hd, 2, dtype=torch.float32)
    inv = 1.0 / (theta ** (j / hd))
    ang = torch.outer(pos.float(), inv).double()
    c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
    x1, x2 = x[..., : hd // 2], x[..., hd // 2:]
    return torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), dim=-1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd,page,theta", [(4, 2, 16, 16, 1e4), (3, 1, 32, 8, 1e6), (28, 4, 128, 16, 1e6), (5, 5, 48, 4, 5e5),
                                                  (4, 2, 6, 8, 1e4), (3, 1, 250, 4, 1e6)])
def test_rope_cache_write(ops, dtype, nh, nkv, hd, page, theta):
    g = torch.Generator().manual_seed(3)
    lens, ctxs = [5, 1, 11], [0, 37, 6]           # three requests: new tokens, cached before
    T = sum(lens)
    max_blocks = (max(a + b for a, b in zip(lens, ctxs)) + page - 1) // page
    pages = 3 * max_blocks + 2
    qkv = torch.randn(T, (nh + 2 * nkv) * hd, generator=g).to(dtype)
    positions = torch.cat([torch.arange(c, c + n) for n, c in zip(lens, ctxs)]).int()
    token_req = torch.cat([torch.full((n,), r) for r, n in enumerate(lens)]).int()
    perm = torch.randperm(pages - 1, generator=g)[: 3 * max_blocks] + 1
    bt = perm.view(3, max_blocks).int()
    j = torch.arange(0, hd, 2, dtype=torch.float32)
    inv_freq = (1.0 / (theta ** (j / hd)))
    kp = torch.zeros(pages, nkv, page, hd, dtype=dtype)
    vp = torch.zeros(pages, nkv, hd, page, dtype=dtype)         # values lie transposed inside a page
    d_qkv, d_kp, d_vp = qkv.cuda(), kp.cuda(), vp.cuda()
    ops.rope_cache_write(d_qkv, nh, nkv, hd, nh + nkv, positions.cuda(), inv_freq.cuda(), token_req.cuda(), bt.cuda(), d_kp, d_vp, page)
    x = qkv.double().view(T, nh + 2 * nkv, hd)
    ref_qk = _rope_ref(x[:, : nh + nkv], positions, theta)
    got = d_qkv.cpu().double().view(T, nh + 2 * nkv, hd)
    torch.testing.assert_close(got[:, : nh + nkv], ref_qk, **_tol(dtype))
    assert torch.equal(got[:, nh + nkv:], x[:, nh + nkv:])
    kref = torch.zeros(pages, nkv, page, hd, dtype=torch.float64)
    vref = torch.zeros(pages, nkv, hd, page, dtype=torch.float64)
    for t in range(T):
        p = int(positions[t]); pg = int(bt[token_req[t], p // page])
        kref[pg, :, p % page] = got[t, nh: nh + nkv]       # the rotated k as stored in place
        vref[pg, :, :, p % page] = x[t, nh + nkv:]
    assert torch.equal(d_kp.cpu().double(), kref)
    assert torch.equal(d_vp.cpu().double(), vref)
    assert float(d_kp[0].abs().sum()) == 0.0                # page 0 is never written


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("lens", [[5, 1, 11], [70, 1, 130]])
@pytest.mark.parametrize("nh,nkv,hd,page,theta", [(4, 2, 16, 16, 1e4), (28, 4, 128, 16, 1e6), (5, 5, 48, 4, 5e5)])
def test_rope_cache_write_in_the_pair_layout(ops, dtype, lens, nh, nkv, hd, page, theta):
    """With the dimensions of every head reordered so that the two that a frequency turns are
    neighbours, the kernel's pair mode gives the reordered result of the usual rotation (a few
    tokens: one wave per head; many tokens in bfloat16: the kernel that moves 16 bytes at a time)."""
    g = torch.Generator().manual_seed(6)
    ctxs = [0, 37, 6]
    T = sum(lens)
    max_blocks = (max(a + b for a, b in zip(lens, ctxs)) + page - 1) // page
    pages = 3 * max_blocks + 2
    qkv = torch.randn(T, (nh + 2 * nkv) * hd, generator=g).to(dtype)
    positions = torch.cat([torch.arange(c, c + n) for n, c in zip(lens, ctxs)]).int()
    token_req = torch.cat([torch.full((n,), r) for r, n in enumerate(lens)]).int()
    bt = (torch.randperm(pages - 1, generator=g)[: 3 * max_blocks] + 1).view(3, max_blocks).int()
    inv_freq = 1.0 / (theta ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd))
    order = torch.cat((ops.pair_layout_rows(nh + nkv, hd), (nh + nkv) * hd + torch.arange(nkv * hd)))    # values keep their order
    outs = []
    for pairs, src in ((False, qkv), (True, qkv[:, order].contiguous())):
        d_qkv = src.cuda()
        d_kp = torch.zeros(pages, nkv, page, hd, dtype=dtype, device="cuda")
        d_vp = torch.zeros(pages, nkv, hd, page, dtype=dtype, device="cuda")
        ops.rope_cache_write(d_qkv, nh, nkv, hd, nh + nkv, positions.cuda(), inv_freq.cuda(), token_req.cuda(), bt.cuda(), d_kp, d_vp, page, pairs=pairs)
        outs.append((d_qkv.cpu(), d_kp.cpu(), d_vp.cpu()))
    (plain_qkv, plain_k, plain_v), (pair_qkv, pair_k, pair_v) = outs
    korder = ops.pair_layout_rows(1, hd)
    assert torch.equal(pair_qkv, plain_qkv[:, order])
    assert torch.equal(pair_k, plain_k[..., korder])
    assert torch.equal(pair_v, plain_v)


@pytest.mark.parametrize("pairs", [False, True])
@pytest.mark.parametrize("nh,nkv,hd,page,P,bias", [(28, 4, 128, 16, 3, True), (4, 2, 16, 8, 1, False), (5, 5, 48, 16, 4, True)])
def test_rope_cache_write_from_slabs_of_partial_sums(ops, pairs, nh, nkv, hd, page, P, bias):
    """The rows come as float slabs of a projection split over K, plus its bias: queries land rotated
    in qkv, rotated keys and values in their pages."""
    g = torch.Generator().manual_seed(8)
    lens, ctxs = [20, 1, 3], [0, 37, 6]
    T = sum(lens)
    width = (nh + 2 * nkv) * hd
    max_blocks = (max(a + b for a, b in zip(lens, ctxs)) + page - 1) // page
    pages = 3 * max_blocks + 2
    parts = torch.randn(P, T, width, generator=g)
    b = torch.randn(width, generator=g).to(torch.bfloat16) if bias else None
    positions = torch.cat([torch.arange(c, c + n) for n, c in zip(lens, ctxs)]).int()
    token_req = torch.cat([torch.full((n,), r) for r, n in enumerate(lens)]).int()
    bt = (torch.randperm(pages - 1, generator=g)[: 3 * max_blocks] + 1).view(3, max_blocks).int()
    inv_freq = 1.0 / (1e5 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd))
    qkv = torch.full((T, width), float("nan"), dtype=torch.bfloat16, device="cuda")
    kp = torch.zeros(pages, nkv, page, hd, dtype=torch.bfloat16, device="cuda")
    vp = torch.zeros(pages, nkv, hd, page, dtype=torch.bfloat16, device="cuda")
    ops.rope_cache_write(qkv, nh, nkv, hd, nh + nkv, positions.cuda(), inv_freq.cuda(), token_req.cuda(), bt.cuda(), kp, vp, page,
                         pairs=pairs, parts=parts.cuda(), bias=None if b is None else b.cuda())
    exact = parts.double().sum(0) + (b.double() if bias else 0.0)
    heads = exact[:, : (nh + nkv) * hd].view(T, nh + nkv, hd)
    ang = (positions.float()[:, None] * inv_freq[None, :]).double()[:, None, :]
    if pairs:
        a, c = heads[..., 0::2], heads[..., 1::2]
        turned = torch.stack((a * ang.cos() - c * ang.sin(), c * ang.cos() + a * ang.sin()), -1).reshape(T, nh + nkv, hd)
    else:
        a, c = heads[..., : hd // 2], heads[..., hd // 2:]
        turned = torch.cat((a * ang.cos() - c * ang.sin(), c * ang.cos() + a * ang.sin()), -1)
    tol = dict(rtol=2 ** -8, atol=1e-5 * float(exact.abs().max()))          # one rounding to bfloat16
    torch.testing.assert_close(qkv[:, : nh * hd].double().cpu(), turned[:, :nh].reshape(T, -1), **tol)
    v = exact[:, (nh + nkv) * hd:].view(T, nkv, hd)
    for t in range(T):
        p = int(positions[t]); pg = int(bt[token_req[t], p // page])
        torch.testing.assert_close(kp[pg, :, p % page].double().cpu(), turned[t, nh:], **tol)
        torch.testing.assert_close(vp[pg, :, :, p % page].double().cpu(), v[t], **tol)
    assert float(kp[0].abs().sum()) == 0.0


@pytest.mark.parametrize("M", [1, 2, 8, 16])
@pytest.mark.parametrize("nh,nkv,hd,page,hidden,bias", [(28, 4, 128, 16, 3584, True), (4, 2, 16, 8, 64, False), (14, 2, 64, 16, 896, True),
                                                        (40, 8, 128, 32, 5120, True), (5, 5, 48, 16, 240, True)])
def test_projection_with_rotation_and_cache_write_in_its_epilogue(ops, M, nh, nkv, hd, page, hidden, bias):
    """The fused query/key/value projection of a decode step against the product, the rotation and
    the cache write done one after the other."""
    g = torch.Generator().manual_seed(M + nh)
    T = M
    ctxs = [int(c) for c in torch.randint(0, 90, (T,), generator=g)]
    max_blocks = (max(ctxs) + 1 + page - 1) // page
    pages = T * max_blocks + 2
    width = (nh + 2 * nkv) * hd
    x = torch.randn(T, hidden, generator=g).to(torch.bfloat16).cuda()
    w = (torch.randn(width, hidden, generator=g) / math.sqrt(hidden)).to(torch.bfloat16).cuda()
    b = torch.randn(width, generator=g).to(torch.bfloat16).cuda() if bias else None
    positions = torch.tensor(ctxs, dtype=torch.int32).cuda()
    token_req = torch.arange(T, dtype=torch.int32).cuda()
    bt = (torch.randperm(pages - 1, generator=g)[: T * max_blocks] + 1).view(T, max_blocks).int().cuda()
    inv_freq = (1.0 / (1e6 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd))).cuda()

    def planes():
        return (torch.zeros(pages, nkv, page, hd, dtype=torch.bfloat16, device="cuda"),
                torch.zeros(pages, nkv, hd, page, dtype=torch.bfloat16, device="cuda"))
    ref = torch.empty(T, width, dtype=torch.bfloat16, device="cuda")
    ops.linear(x, w, b, ref)
    rk, rv = planes()
    ops.rope_cache_write(ref, nh, nkv, hd, nh + nkv, positions, inv_freq, token_req, bt, rk, rv, page, pairs=True)
    got = torch.full((T, width), float("nan"), dtype=torch.bfloat16, device="cuda")
    gk, gv = planes()
    fused = ops.linear_rope_cache_write(x, w, b, got, nh, nkv, hd, positions, inv_freq, token_req, bt, gk, gv, page)
    # from 9 rows on the library declines where the product split over K plus the rotation kernel is ahead
    assert fused == (M <= 8 or not ops.linear_partials_pay(M, width, hidden))
    if not fused:
        return
    # against the exact product and rotation: the fused kernel rounds once, to bfloat16, at the end
    # (half an ulp, 2^-9 of the value; 2^-8 allowed), on top of the 32-bit sums' own error
    exact = x.double().cpu() @ w.double().cpu().T + (b.double().cpu() if bias else 0.0)
    heads = exact[:, : (nh + nkv) * hd].view(T, nh + nkv, hd)
    ang = (positions.cpu().float()[:, None] * inv_freq.cpu()[None, :]).double()[:, None, :]
    a, c = heads[..., 0::2], heads[..., 1::2]
    turned = torch.stack((a * ang.cos() - c * ang.sin(), c * ang.cos() + a * ang.sin()), -1).reshape(T, nh + nkv, hd)
    tol = dict(rtol=2 ** -8, atol=1e-5 * float(exact.abs().max()))
    torch.testing.assert_close(got[:, : nh * hd].double().cpu(), turned[:, :nh].reshape(T, -1), **tol)
    for t in range(T):
        pg, off = int(bt[t, ctxs[t] // page]), ctxs[t] % page
        torch.testing.assert_close(gk[pg, :, off].double().cpu(), turned[t, nh:], **tol)
    # and next to the two-kernel path, which rounds twice: a whole ulp apart at most
    loose = dict(rtol=2 ** -6, atol=2 ** -7 * float(exact.abs().max()))
    torch.testing.assert_close(got[:, : nh * hd].float(), ref[:, : nh * hd].float(), **loose)
    torch.testing.assert_close(gk.float(), rk.float(), **loose)
    assert torch.equal(gv, rv)
    assert float(gk[0].abs().sum()) == 0.0 and float(gv[0].abs().sum()) == 0.0
    # queries alone, as a run that reads another run's cache asks for them
    q_only = torch.empty(T, nh * hd, dtype=torch.bfloat16, device="cuda")
    assert ops.linear_rope_cache_write(x, w[: nh * hd], None if b is None else b[: nh * hd], q_only, nh, nkv, hd, positions, inv_freq)
    assert torch.equal(q_only, got[:, : nh * hd])


@pytest.mark.parametrize("rows,hidden", [(1, 96), (3, 3584), (5, 5120), (2, 1000), (2, 20000)])
@pytest.mark.parametrize("slabs", [1, 2, 3, 4, 5, 6, 7, 9])
def test_add_rmsnorm_adds_any_number_of_slabs_in_their_order(ops, rows, hidden, slabs):
    """The pending branch as float slabs of partial sums: four are fetched at a time, the last one to three as a
    group of their own; the new residual is the sum in the slabs' order, to the bit."""
    g = torch.Generator().manual_seed(rows * hidden + slabs)
    res = torch.randn(rows, hidden, generator=g)
    parts = torch.randn(slabs, rows, hidden, generator=g)
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(torch.bfloat16)
    total = res.clone()
    for p in range(slabs):
        total = total + parts[p]                      # 32-bit, in this order
    r = res.clone().cuda()
    out = torch.empty(rows, hidden, dtype=torch.bfloat16, device="cuda")
    ops.add_rmsnorm(r, parts.cuda(), w.cuda(), 1e-6, out)
    assert torch.equal(r.cpu(), total)
    ref = total.double() * torch.rsqrt(total.double().pow(2).mean(-1, keepdim=True) + 1e-6) * w.double()
    torch.testing.assert_close(out.cpu().double(), ref, **_tol(torch.bfloat16))


@pytest.mark.parametrize("H,I", [(96, 200), (3584, 1000), (1032, 300), (5120, 512), (8192, 96)])
@pytest.mark.parametrize("pending", ["none", "row", "slabs"])
@pytest.mark.parametrize("wdtype", [torch.bfloat16, torch.float32])
def test_gate_up_product_of_one_row_that_makes_its_norm_itself(ops, H, I, pending, wdtype):
    """``linear_swiglu_normed`` against the norm's own kernel followed by ``linear_swiglu``: the new
    residual to the bit, the product within the rounding of one more order of summation."""
    g = torch.Generator().manual_seed(H + I)
    res = torch.randn(1, H, generator=g).cuda()
    w = (1 + 0.1 * torch.randn(H, generator=g)).to(wdtype).cuda()
    pend = {"none": None, "row": torch.randn(1, H, generator=g).to(torch.bfloat16).cuda(),
            "slabs": torch.randn(3, 1, H, generator=g).cuda()}[pending]
    gate = (torch.randn(I, H, generator=g) / math.sqrt(H)).to(torch.bfloat16).cuda()
    up = (torch.randn(I, H, generator=g) / math.sqrt(H)).to(torch.bfloat16).cuda()
    gu = ops.interleave_gate_up(gate, up)
    r0, h = res.clone(), torch.empty(1, H, dtype=torch.bfloat16, device="cuda")
    ops.add_rmsnorm(r0, pend, w, 1e-5, h)
    z0 = torch.empty(1, I, dtype=torch.bfloat16, device="cuda")
    ops.linear_swiglu(h, gu, z0)
    z1 = torch.full((1, I), float("nan"), dtype=torch.bfloat16, device="cuda")
    rout = torch.full_like(res, float("nan"))
    assert ops.linear_swiglu_normed(res, pend, w, 1e-5, rout, gu, z1)
    assert torch.equal(rout, r0)
    torch.testing.assert_close(z1.float(), z0.float(), **_tol(torch.bfloat16))
    # what it is not built for it declines, leaving everything alone
    long = torch.randn(1, 16384 + 64, generator=g).cuda()
    gul = torch.zeros(64, 16384 + 64, dtype=torch.bfloat16, device="cuda")
    zl = torch.empty(1, 32, dtype=torch.bfloat16, device="cuda")
    assert not ops.linear_swiglu_normed(long, None, torch.ones(16384 + 64, dtype=wdtype, device="cuda"), 1e-5, torch.empty_like(long), gul, zl)
    assert not ops.linear_swiglu_normed(torch.randn(2, H).cuda(), None, w, 1e-5, torch.empty(2, H).cuda(), gu, torch.empty(2, I, dtype=torch.bfloat16, device="cuda"))


@pytest.mark.parametrize("nh,nkv,hd,page,hidden,bias", [(28, 4, 128, 16, 3584, True), (4, 2, 16, 8, 64, False), (14, 2, 64, 16, 896, True),
                                                        (40, 8, 128, 32, 5120, True), (5, 5, 48, 16, 240, True)])
@pytest.mark.parametrize("pending", ["none", "row", "slabs", "1 slab", "3 slabs", "7 slabs", "8 slabs"])
def test_projection_of_one_row_that_makes_its_norm_itself(ops, nh, nkv, hd, page, hidden, bias, pending):
    """``linear_rope_cache_write_normed`` against the norm's own kernel followed by the fused projection:
    the new residual, the rotated queries and what lands in the pages, to the bit (slabs of partial sums are
    fetched four at a time, the last one to three as a group of their own)."""
    g = torch.Generator().manual_seed(nh + hidden)
    width = (nh + 2 * nkv) * hd
    res = torch.randn(1, hidden, generator=g).cuda()
    nw = (1 + 0.1 * torch.randn(hidden, generator=g)).to(torch.bfloat16).cuda()
    if pending == "none":
        pend = None
    elif pending == "row":
        pend = torch.randn(1, hidden, generator=g).to(torch.bfloat16).cuda()
    else:
        pend = torch.randn(4 if pending == "slabs" else int(pending.split()[0]), 1, hidden, generator=g).cuda()
    w = (torch.randn(width, hidden, generator=g) / math.sqrt(hidden)).to(torch.bfloat16).cuda()
    b = torch.randn(width, generator=g).to(torch.bfloat16).cuda() if bias else None
    inv_freq = (1.0 / (1e6 ** (torch.arange(0, hd, 2).float() / hd))).cuda()
    pos = 77
    positions = torch.tensor([pos], dtype=torch.int32).cuda()
    token_req = torch.zeros(1, dtype=torch.int32).cuda()
    blocks = pos // page + 1
    bt = (torch.arange(blocks, dtype=torch.int32) + 1).view(1, blocks).cuda()

    def planes():
        return (torch.zeros(blocks + 1, nkv, page, hd, dtype=torch.bfloat16, device="cuda"),
                torch.zeros(blocks + 1, nkv, hd, page, dtype=torch.bfloat16, device="cuda"))
    r0, h = res.clone(), torch.empty(1, hidden, dtype=torch.bfloat16, device="cuda")
    ops.add_rmsnorm(r0, pend, nw, 1e-6, h)
    k0, v0 = planes()
    q0 = torch.empty(1, width, dtype=torch.bfloat16, device="cuda")
    assert ops.linear_rope_cache_write(h, w, b, q0, nh, nkv, hd, positions, inv_freq, token_req, bt, k0, v0, page)
    k1, v1 = planes()
    q1 = torch.full((1, width), float("nan"), dtype=torch.bfloat16, device="cuda")
    rout = torch.full_like(res, float("nan"))
    assert ops.linear_rope_cache_write_normed(res, pend, nw, 1e-6, rout, w, b, q1, nh, nkv, hd, positions, inv_freq,
                                              token_req, bt, k1, v1, page)
    assert torch.equal(rout, r0)
    assert torch.equal(q1[:, : nh * hd], q0[:, : nh * hd]) and torch.equal(k1, k0) and torch.equal(v1, v0)
    assert float(k1[0].abs().sum()) == 0.0


def _attention_ref(q, k, v, window):
    """One request: q [n, heads, hd] at positions ctx..ctx+n-1, k/v [ctx+n, kvh, hd] (float64)."""
    n, heads, hd = q.shape
    total, kvh, _ = k.shape
    ctx = total - n
    group = heads // kvh
    kk = k.repeat_interleave(group, dim=1)
    vv = v.repeat_interleave(group, dim=1)
    s = torch.einsum("nhd,thd->hnt", q, kk) / math.sqrt(hd)
    qpos = ctx + torch.arange(n)[:, None]
    kpos = torch.arange(total)[None, :]
    hide = kpos > qpos
    if window:
        hide = hide | (kpos <= qpos - window)
    s = s.masked_fill(hide[None], -torch.inf)
    return torch.einsum("hnt,thd->nhd", torch.softmax(s, -1), vv)


@pytest.mark.parametrize("dtype,general,waves", [(torch.float32, False, 4), (torch.bfloat16, False, 4), (torch.bfloat16, False, 8), (torch.bfloat16, True, 4)])
@pytest.mark.parametrize("nh,nkv,hd,page,window,splits", [
    (4, 2, 16, 16, 0, 1), (3, 1, 32, 8, 0, 1), (28, 4, 128, 16, 0, 3), (6, 6, 48, 4, 0, 1),
    (20, 1, 64, 16, 0, 2), (4, 2, 16, 16, 13, 1), (8, 2, 80, 32, 29, 4), (2, 1, 256, 16, 0, 1),
    (5, 5, 32, 2, 0, 2), (14, 2, 128, 64, 40, 5),
    (4, 2, 4, 4, 0, 1), (10, 2, 24, 16, 0, 3), (3, 3, 250, 8, 17, 2), (5, 1, 40, 16, 0, 2), (2, 1, 2, 16, 0, 1),
])
def test_paged_attention(ops, dtype, general, waves, nh, nkv, hd, page, window, splits):
    """float32 and bfloat16 through the general kernel, bfloat16 through the matrix-core kernel
    (pages of 2 tokens fall back to the general one by themselves, and so do head sizes that are
    no multiple of 16: the library of the next multiple serves them)."""
    g = torch.Generator().manual_seed(4)
    lens, ctxs = [37, 1, 9, 1], [0, 150, 70, 0]      # a whole prompt, a decode, a portion, a first token
    R, T = len(lens), sum(lens)
    totals = [a + b for a, b in zip(lens, ctxs)]
    max_blocks = (max(totals) + page - 1) // page + 1
    pages = R * max_blocks + 1
    bt = (torch.randperm(pages - 1, generator=g)[: R * max_blocks] + 1).view(R, max_blocks).int()
    q = torch.randn(T, nh * hd, generator=g).to(dtype)
    # places that hold no key yet are NaN (a page that another request left behind may hold anything):
    # nothing of them may reach a result
    kp = torch.full((pages, nkv, page, hd), float("nan"), dtype=dtype)
    vp = torch.full((pages, nkv, hd, page), float("nan"), dtype=dtype)      # transposed inside a page
    ks, vs = [], []
    for r in range(R):
        k = torch.randn(totals[r], nkv, hd, generator=g).to(dtype)
        v = torch.randn(totals[r], nkv, hd, generator=g).to(dtype)
        if r == 0:
            k[3] *= 4.0        # a far key stands out: dropping it changes the result visibly
        for p in range(totals[r]):
            kp[bt[r, p // page], :, p % page] = k[p]
            vp[bt[r, p // page], :, :, p % page] = v[p]
        ks.append(k); vs.append(v)
    indptr = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    tq = ops.attention_tile_tokens(nh, nkv)
    tile_req, tile_tok0 = [], []
    for r, n in enumerate(lens):
        for t0 in range(0, n, tq):
            tile_req.append(r); tile_tok0.append(t0)
    out = torch.empty(T, nh * hd, dtype=dtype, device="cuda")
    # q lives inside a wider row, as in the fused projection
    wide = torch.zeros(T, nh * hd + 32, dtype=dtype, device="cuda")
    wide[:, : nh * hd] = q.cuda()
    ops.paged_attention(wide[:, : nh * hd], out, kp.cuda(), vp.cuda(), bt.cuda(), indptr.cuda(),
                        torch.tensor(ctxs, dtype=torch.int32).cuda(), torch.tensor(tile_req, dtype=torch.int32).cuda(),
                        torch.tensor(tile_tok0, dtype=torch.int32).cuda(), len(tile_req), tq, nh, nkv, hd, page, window,
                        1.0 / math.sqrt(hd), splits, general=general, waves=waves)
    got = out.cpu().double().view(T, nh, hd)
    for r in range(R):
        a, b = int(indptr[r]), int(indptr[r + 1])
        ref = _attention_ref(q[a:b].double().view(-1, nh, hd), ks[r].double(), vs[r].double(), window)
        tol = _tol(dtype)
        if dtype == torch.bfloat16 and not general:
            # the matrix-core kernel rounds the probabilities to bfloat16 before the product with V
            # (half an ulp, 2^-9 of each weight), on top of the rounding of the result
            tol = dict(rtol=tol["rtol"], atol=tol["atol"] + 2 ** -9 * float(vs[r].abs().max()))
        torch.testing.assert_close(got[a:b], ref, **tol)


@pytest.mark.parametrize("dtype,general", [(torch.float32, False), (torch.bfloat16, False), (torch.bfloat16, True)])
@pytest.mark.parametrize("nh,nkv,hd,page,window,splits,wide", [
    (28, 4, 128, 16, 0, 3, 0), (6, 2, 32, 8, 0, 1, 5), (4, 4, 16, 4, 11, 2, 0), (14, 2, 64, 16, 0, 4, 2100), (5, 1, 48, 32, 40, 1, 3),
])
def test_paged_attention_of_a_decode_step_without_a_tile_list(ops, dtype, general, nh, nkv, hd, page, window, splits, wide):
    """One new token per request and no tile list (the kernel takes tile i for the token of request i and
    asks for length, block table and query at once): the same bits as with the list, for short and long
    contexts, a first token, and a block table wider than the kernel keeps in shared memory."""
    g = torch.Generator().manual_seed(6)
    ctxs = [150, 0, 70, 33, 1, 299]
    R = len(ctxs)
    max_blocks = (max(ctxs) + page) // page + 1 + wide
    pages = R * ((max(ctxs) + page) // page + 1) + 1
    bt = torch.zeros(R, max_blocks, dtype=torch.int32)
    used = (max(ctxs) + page) // page + 1
    bt[:, :used] = (torch.randperm(pages - 1, generator=g)[: R * used] + 1).view(R, used).int()
    q = torch.randn(R, nh * hd, generator=g).to(dtype).cuda()
    kp = torch.randn(pages, nkv, page, hd, generator=g).to(dtype).cuda()
    vp = torch.randn(pages, nkv, hd, page, generator=g).to(dtype).cuda()
    indptr = torch.arange(R + 1, dtype=torch.int32).cuda()
    ctx_t = torch.tensor(ctxs, dtype=torch.int32).cuda()
    tiles = torch.arange(R, dtype=torch.int32).cuda()
    zeros = torch.zeros(R, dtype=torch.int32).cuda()
    tq = ops.attention_tile_tokens(nh, nkv)
    common = (nh, nkv, hd, page, window, 1.0 / math.sqrt(hd), splits)
    listed = torch.empty(R, nh * hd, dtype=dtype, device="cuda")
    ops.paged_attention(q, listed, kp, vp, bt.cuda(), indptr, ctx_t, tiles, zeros, R, tq, *common, general=general)
    bare = torch.full_like(listed, float("nan"))
    ops.paged_attention(q, bare, kp, vp, bt.cuda(), None, ctx_t, None, None, R, tq, *common, general=general)
    assert torch.equal(bare, listed) and bool(torch.isfinite(bare.float()).all())
    with pytest.raises(ops.KernelError, match="exactly one token"):
        ops.paged_attention(q, bare, kp, vp, bt.cuda(), None, ctx_t, None, None, R - 1, tq, *common, general=general)


@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_of_some_requests_leaves_the_other_rows_alone(ops, dtype):
    """Tiles of two of four requests, keys split over work-groups: with the tokens of those
    requests listed, the merge of the parts writes their rows only."""
    nh, nkv, hd, page, splits = 6, 2, 32, 8, 3
    g = torch.Generator().manual_seed(9)
    lens, ctxs = [5, 1, 40, 1], [60, 150, 0, 90]
    chosen = [1, 3]
    R, T = len(lens), sum(lens)
    totals = [a + b for a, b in zip(lens, ctxs)]
    max_blocks = (max(totals) + page - 1) // page + 1
    pages = R * max_blocks + 1
    bt = (torch.randperm(pages - 1, generator=g)[: R * max_blocks] + 1).view(R, max_blocks).int()
    q = torch.randn(T, nh * hd, generator=g).to(dtype)
    kp = torch.randn(pages, nkv, page, hd, generator=g).to(dtype)
    vp = torch.randn(pages, nkv, hd, page, generator=g).to(dtype)
    ks, vs = [], []
    for r in range(R):
        k = torch.randn(totals[r], nkv, hd, generator=g).to(dtype)
        v = torch.randn(totals[r], nkv, hd, generator=g).to(dtype)
        for p in range(totals[r]):
            kp[bt[r, p // page], :, p % page] = k[p]
            vp[bt[r, p // page], :, :, p % page] = v[p]
        ks.append(k); vs.append(v)
    indptr = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    tq = ops.attention_tile_tokens(nh, nkv)
    tile_req = [r for r in chosen for _ in range(0, lens[r], tq)]
    tile_tok0 = [t0 for r in chosen for t0 in range(0, lens[r], tq)]
    tokens = [t for r in chosen for t in range(int(indptr[r]), int(indptr[r + 1]))]
    out = torch.full((T, nh * hd), 7.0, dtype=dtype, device="cuda")
    ops.paged_attention(q.cuda(), out, kp.cuda(), vp.cuda(), bt.cuda(), indptr.cuda(),
                        torch.tensor(ctxs, dtype=torch.int32).cuda(), torch.tensor(tile_req, dtype=torch.int32).cuda(),
                        torch.tensor(tile_tok0, dtype=torch.int32).cuda(), len(tile_req), tq, nh, nkv, hd, page, 0,
                        1.0 / math.sqrt(hd), splits, merge_tokens=(torch.tensor(tokens, dtype=torch.int32).cuda(), len(tokens)))
    got = out.cpu().double().view(T, nh, hd)
    for r in range(R):
        a, b = int(indptr[r]), int(indptr[r + 1])
        if r in chosen:
            ref = _attention_ref(q[a:b].double().view(-1, nh, hd), ks[r].double(), vs[r].double(), 0)
            tol = _tol(dtype)
            torch.testing.assert_close(got[a:b], ref, rtol=tol["rtol"], atol=tol["atol"] + 2 ** -9 * float(vs[r].abs().max()))
        else:
            assert bool((got[a:b] == 7.0).all()), f"rows of request {r} were written"


@pytest.mark.parametrize("nh,nkv,hd,page,window", [
    (4, 2, 16, 16, 0), (3, 1, 32, 8, 0), (28, 4, 128, 16, 0), (6, 6, 48, 4, 0), (20, 1, 64, 16, 0),
    (4, 2, 16, 16, 13), (8, 2, 80, 32, 29), (14, 2, 128, 64, 40), (5, 5, 112, 12, 70),
])
def test_paged_attention_prompt_portions(ops, nh, nkv, hd, page, window):
    """The shared-memory kernel for prompt portions: whole prompts, portions on top of a cached
    context (also one that starts inside a page and inside a 32-key chunk), a single token."""
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(14)
    lens, ctxs = [150, 37, 70, 1, 64], [0, 150, 43, 99, 64]
    R, T = len(lens), sum(lens)
    totals = [a + b for a, b in zip(lens, ctxs)]
    max_blocks = (max(totals) + page - 1) // page + 1
    pages = R * max_blocks + 1
    bt = (torch.randperm(pages - 1, generator=g)[: R * max_blocks] + 1).view(R, max_blocks).int()
    q = torch.randn(T, nh * hd, generator=g).to(dtype)
    kp = torch.full((pages, nkv, page, hd), float("nan"), dtype=dtype)      # NaN where no key is written
    vp = torch.full((pages, nkv, hd, page), float("nan"), dtype=dtype)
    ks, vs = [], []
    for r in range(R):
        k = torch.randn(totals[r], nkv, hd, generator=g).to(dtype)
        v = torch.randn(totals[r], nkv, hd, generator=g).to(dtype)
        k[min(3, totals[r] - 1)] *= 3.0
        for p in range(totals[r]):
            kp[bt[r, p // page], :, p % page] = k[p]
            vp[bt[r, p // page], :, :, p % page] = v[p]
        ks.append(k); vs.append(v)
    indptr = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    tq = ops.prefill_attention_tile_tokens(nh, nkv)
    tile_req, tile_tok0 = [], []
    for r, n in enumerate(lens):
        for t0 in range(0, n, tq):
            tile_req.append(r); tile_tok0.append(t0)
    out = torch.full((T, nh * hd), float("nan"), dtype=dtype, device="cuda")
    wide = torch.zeros(T, nh * hd + 32, dtype=dtype, device="cuda")
    wide[:, : nh * hd] = q.cuda()
    ops.paged_attention_prefill(wide[:, : nh * hd], out, kp.cuda(), vp.cuda(), bt.cuda(), indptr.cuda(),
                                torch.tensor(ctxs, dtype=torch.int32).cuda(), torch.tensor(tile_req, dtype=torch.int32).cuda(),
                                torch.tensor(tile_tok0, dtype=torch.int32).cuda(), len(tile_req), tq, nh, nkv, hd, page, window,
                                1.0 / math.sqrt(hd))
    got = out.cpu().double().view(T, nh, hd)
    for r in range(R):
        a, b = int(indptr[r]), int(indptr[r + 1])
        ref = _attention_ref(q[a:b].double().view(-1, nh, hd), ks[r].double(), vs[r].double(), window)
        tol = _tol(dtype)
        tol = dict(rtol=tol["rtol"], atol=tol["atol"] + 2 ** -9 * float(vs[r].abs().max()))
        torch.testing.assert_close(got[a:b], ref, **tol)


@pytest.mark.parametrize("nh,nkv,hd,page,window", [
    (28, 4, 128, 16, 0), (20, 1, 64, 16, 0), (40, 8, 128, 8, 0), (4, 4, 64, 32, 0), (130, 1, 64, 16, 0),
    (14, 2, 128, 64, 40), (4, 4, 64, 32, 29), (6, 2, 128, 8, 100),
    (28, 4, 128, 128, 0), (6, 2, 64, 256, 100),              # pages longer than a step: steps begin inside a page
])
def test_paged_attention_prompt_tiles_of_128_rows(ops, nh, nkv, hd, page, window):
    """The 128-row kernel for prompt portions: whole prompts, portions on top of a cached context
    (also one that starts inside a page and inside a step of 64 keys), a single token, groups of
    1, 3, 5, 7, 20 and 130 heads.  Places of the pages that hold no key yet are filled with NaN:
    nothing of them may reach a result."""
    assert ops.prompt_attention_fits(torch.bfloat16, hd, page) and not ops.prompt_attention_fits(torch.bfloat16, hd, 24)
    _prompt_tiles_case(ops, nh, nkv, hd, page, window, [150, 37, 70, 1, 64, 300], [0, 150, 43, 99, 64, 5])


def test_paged_attention_prompt_with_more_tiles_than_compute_units_but_no_more_than_fit_at_once(ops):
    """Between one and two work-groups a compute unit the kernel runs its second batch of tiles from light to
    heavy: four requests of different lengths, 96 tiles of 18 tokens for each of 4 key/value heads, and the
    same split over the keys (then the order is the plain one)."""
    nh, nkv = 28, 4
    lens = [700, 500, 300, 200]
    tiles = sum(-(-n // ops.prompt_attention_tile_tokens(nh, nkv)) for n in lens) * nkv
    units = torch.cuda.get_device_properties(0).multi_processor_count
    if not units < tiles <= 2 * units:
        pytest.skip(f"{tiles} work-groups on {units} compute units: not the case this test is for")
    _prompt_tiles_case(ops, nh, nkv, 128, 16, 0, lens, [0, 37, 0, 64])


def _prompt_tiles_case(ops, nh, nkv, hd, page, window, lens, ctxs):
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(15)
    R, T = len(lens), sum(lens)
    totals = [a + b for a, b in zip(lens, ctxs)]
    max_blocks = (max(totals) + page - 1) // page + 1
    pages = R * max_blocks + 1
    bt = (torch.randperm(pages - 1, generator=g)[: R * max_blocks] + 1).view(R, max_blocks).int()
    q = torch.randn(T, nh * hd, generator=g).to(dtype)
    kp = torch.full((pages, nkv, page, hd), float("nan"), dtype=dtype)
    vp = torch.full((pages, nkv, hd, page), float("nan"), dtype=dtype)
    ks, vs = [], []
    for r in range(R):
        k = torch.randn(totals[r], nkv, hd, generator=g).to(dtype)
        v = torch.randn(totals[r], nkv, hd, generator=g).to(dtype)
        k[min(3, totals[r] - 1)] *= 3.0
        for p in range(totals[r]):
            kp[bt[r, p // page], :, p % page] = k[p]
            vp[bt[r, p // page], :, :, p % page] = v[p]
        ks.append(k); vs.append(v)
    indptr = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    tq = ops.prompt_attention_tile_tokens(nh, nkv)
    tile_req, tile_tok0 = [], []
    for r, n in enumerate(lens):
        for t0 in range(0, n, tq):
            tile_req.append(r); tile_tok0.append(t0)
    out = torch.full((T, nh * hd), float("nan"), dtype=dtype, device="cuda")
    wide = torch.zeros(T, nh * hd + 32, dtype=dtype, device="cuda")
    wide[:, : nh * hd] = q.cuda()
    args = (kp.cuda(), vp.cuda(), bt.cuda(), indptr.cuda(),
            torch.tensor(ctxs, dtype=torch.int32).cuda(), torch.tensor(tile_req, dtype=torch.int32).cuda(),
            torch.tensor(tile_tok0, dtype=torch.int32).cuda(), len(tile_req), tq, nh, nkv, hd, page, window,
            1.0 / math.sqrt(hd))
    ops.paged_attention_prompt(wide[:, : nh * hd], out, *args)
    # the same with every tile's keys dealt to two, three and five work-groups (some shares are empty:
    # the single token has 100 keys, four steps of 32) and merged for all tokens but those of request 2
    listed = [t for r in range(R) if r != 2 for t in range(int(indptr[r]), int(indptr[r + 1]))]
    keep = [i for i, r in enumerate(tile_req) if r != 2]
    some = (args[0], args[1], args[2], args[3], args[4], torch.tensor([tile_req[i] for i in keep], dtype=torch.int32).cuda(),
            torch.tensor([tile_tok0[i] for i in keep], dtype=torch.int32).cuda(), len(keep)) + args[8:]
    outs = [out]
    for splits in (2, 3, 5):
        o = torch.full((T, nh * hd), 9.0, dtype=dtype, device="cuda")
        ops.paged_attention_prompt(wide[:, : nh * hd], o, *some, splits=splits,
                                   merge_tokens=(torch.tensor(listed, dtype=torch.int32).cuda(), len(listed)))
        a2, b2 = int(indptr[2]), int(indptr[3])
        assert bool((o[a2:b2] == 9.0).all()), "rows of a request outside the list were written"
        outs.append(o)
    for k, o in enumerate(outs):
        got = o.cpu().double().view(T, nh, hd)
        for r in range(R):
            if k and r == 2:
                continue
            a, b = int(indptr[r]), int(indptr[r + 1])
            ref = _attention_ref(q[a:b].double().view(-1, nh, hd), ks[r].double(), vs[r].double(), window)
            tol = _tol(dtype)
            tol = dict(rtol=tol["rtol"], atol=tol["atol"] + 2 ** -9 * float(vs[r].abs().max()))
            torch.testing.assert_close(got[a:b], ref, **tol)


def test_paged_attention_prompt_takes_a_wide_block_table_for_short_sequences(ops):
    """What bounds the 128-row kernel is the longest sequence of the step in pages, not the
    room that the block table has: a table of 5000 entries holds a sequence of 200 tokens, and
    a step that says it holds a sequence of 2049 pages is refused before any launch."""
    nh, nkv, hd, page = 4, 2, 64, 8
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(16)
    n = 200
    bt = torch.zeros(1, 5000, dtype=torch.int32)
    used = (n + page - 1) // page
    bt[0, :used] = torch.randperm(used, generator=g).int() + 1
    q = torch.randn(n, nh * hd, generator=g).to(dtype)
    k = torch.randn(n, nkv, hd, generator=g).to(dtype)
    v = torch.randn(n, nkv, hd, generator=g).to(dtype)
    kp = torch.zeros(used + 1, nkv, page, hd, dtype=dtype)
    vp = torch.zeros(used + 1, nkv, hd, page, dtype=dtype)
    for p in range(n):
        kp[bt[0, p // page], :, p % page] = k[p]
        vp[bt[0, p // page], :, :, p % page] = v[p]
    tq = ops.prompt_attention_tile_tokens(nh, nkv)
    tile_tok0 = list(range(0, n, tq))
    args = (kp.cuda(), vp.cuda(), bt.cuda(), torch.tensor([0, n], dtype=torch.int32).cuda(),
            torch.zeros(1, dtype=torch.int32).cuda(), torch.zeros(len(tile_tok0), dtype=torch.int32).cuda(),
            torch.tensor(tile_tok0, dtype=torch.int32).cuda(), len(tile_tok0), tq, nh, nkv, hd, page, 0, 1.0 / math.sqrt(hd))
    out = torch.full((n, nh * hd), float("nan"), dtype=dtype, device="cuda")
    with pytest.raises(ops.KernelError, match="2048 pages"):
        ops.paged_attention_prompt(q.cuda(), out, *args)                     # as long as the table is wide, for all the kernel knows
    with pytest.raises(ops.KernelError, match="2048 pages"):
        ops.paged_attention_prompt(q.cuda(), out, *args, max_total_len=2049 * page)
    ops.paged_attention_prompt(q.cuda(), out, *args, max_total_len=n)
    ref = _attention_ref(q.double().view(-1, nh, hd), k.double(), v.double(), 0)
    tol = _tol(dtype)
    torch.testing.assert_close(out.cpu().double().view(n, nh, hd), ref, rtol=tol["rtol"],
                               atol=tol["atol"] + 2 ** -9 * float(v.abs().max()))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,I", [(3, 200), (17, 1001)])
def test_swiglu(ops, dtype, T, I):
    g = torch.Generator().manual_seed(5)
    gu = (torch.randn(T, 2 * I, generator=g) * 3).to(dtype).cuda()
    out = torch.empty(T, I, dtype=dtype, device="cuda")
    ops.swiglu(gu, out)
    ref = torch.nn.functional.silu(gu[:, :I].double()) * gu[:, I:].double()
    torch.testing.assert_close(out.double(), ref, **_tol(dtype))


def _mix32(x):
    x &= 0xFFFFFFFF
    x ^= x >> 16; x = (x * 0x7FEB352D) & 0xFFFFFFFF
    x ^= x >> 15; x = (x * 0x846CA68B) & 0xFFFFFFFF
    x ^= x >> 16
    return x


def test_sample_greedy_and_ties(ops):
    g = torch.Generator().manual_seed(6)
    logits = torch.randn(5, 3001, generator=g)
    logits[1, 77] = logits[1, 2900] = 50.0          # a tie: the lower index wins
    logits[2, 3000] = 60.0                          # the last column
    out = torch.empty(5, dtype=torch.int32, device="cuda")
    ops.sample(logits.cuda(), None, None, out)
    ref = logits.argmax(-1)
    ref[1] = 77
    assert out.cpu().tolist() == ref.tolist()
    wide = torch.zeros(5, 3100)
    wide[:, :3001] = logits
    wide[:, 3001:] = 1000.0                         # beyond the vocabulary: never read
    ops.sample(wide.cuda()[:, :3001], torch.zeros(5).cuda(), torch.arange(5, dtype=torch.int32).cuda(), out)
    assert out.cpu().tolist() == ref.tolist()


def test_sample_temperature_matches_formula_and_distribution(ops):
    V = 11
    logits = torch.tensor([[0.0, 1.0, 2.0, -1.0, 0.5, 3.0, -2.0, 0.0, 1.5, 2.5, -0.5]])
    temp = 0.8
    n = 20000
    keys = torch.arange(n, dtype=torch.int64)
    keys = ((keys * 2654435761) % (1 << 32)).to(torch.int64)
    keys_i32 = torch.where(keys >= (1 << 31), keys - (1 << 32), keys).int()
    out = torch.empty(n, dtype=torch.int32, device="cuda")
    ops.sample(logits.expand(n, V).contiguous().cuda(), torch.full((n,), temp).cuda(), keys_i32.cuda(), out)
    got = out.cpu()
    # the documented formula, for the first rows, in float64
    for row in range(50):
        key = int(keys[row])
        best, besti = -math.inf, -1
        for i in range(V):
            r = _mix32(_mix32(key ^ i) + 0x9E3779B9)
            u = ((r >> 8) + 0.5) / 16777216.0
            v = float(logits[0, i]) / temp - math.log(-math.log(u))
            if v > best:
                best, besti = v, i
        assert int(got[row]) == besti
    freq = torch.bincount(got.long(), minlength=V).double() / n
    p = torch.softmax(logits[0].double() / temp, -1)
    # 20000 draws: standard error of a frequency is at most 0.0035; allow 4 of them
    assert float((freq - p).abs().max()) < 0.015


def test_stream_read_reads_every_word(ops):
    """The benchmark's yardstick kernel folds every 32-bit word it reads into its result: flipping one bit
    anywhere flips the result, for sizes that are no multiple of anything."""
    import numpy as np
    g = torch.Generator().manual_seed(12)
    fold = lambda t: int(np.bitwise_xor.reduce(t.cpu().numpy().view("uint32")))
    for words in (4, 1000, 256 * 8 * 4 * 64 + 4, 5_000_004):
        data = torch.randint(-2 ** 31, 2 ** 31 - 1, (words,), generator=g, dtype=torch.int64).to(torch.int32).cuda()
        used = words // 4 * 4                     # whole 16-byte pieces
        assert fold(ops.stream_read(data)) == fold(data[:used])
        data[used // 2] ^= 1 << 7
        assert fold(ops.stream_read(data)) == fold(data[:used])
