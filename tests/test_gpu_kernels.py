"""Each HIP kernel alone against a plain torch reference in float64, at sizes other than the
tiny models': odd widths, tails, head sizes in steps of 16, many kv groups, long key ranges."""
import math

import numpy as np
import pytest
import torch

from helpers import PAGE, attention_oracle, fill_kv, make_ctx, make_kv, read_kv

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from libllm_amd.hip import HipOps
    return HipOps()


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


BF16_2ULP = 2.0 ** -7     # two units in the last place of the largest value, for a result rounded once or twice


def max_err(out, ref):
    """max|out - ref| / max|ref|: a bfloat16 result rounded once is within 2^-9 of the largest value."""
    out = torch.as_tensor(out).double().cpu()
    ref = torch.as_tensor(ref).double().cpu()
    return float((out - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


def close(out, ref, dtype, f32=1e-5, bf16=BF16_2ULP):
    return max_err(out, ref) < (f32 if dtype == torch.float32 else bf16)


# ------------------------------------------------------------------------------- embedding
@pytest.mark.parametrize("dtype", DTYPES)
def test_embed(ops, dtype):
    table = rnd((517, 96), dtype, 1).cuda()
    ids = torch.tensor([0, 516, 3, 3, 77, 100], dtype=torch.int32).cuda()
    out = ops.embed(table, ids, 1.0)
    assert out.dtype == torch.float32
    assert torch.equal(out.cpu(), table.float().cpu()[ids.cpu().long()])
    out = ops.embed(table, ids, 2.5)
    assert torch.equal(out.cpu(), table.float().cpu()[ids.cpu().long()] * 2.5)


def test_embed_reference_vector(ops):
    # src/flint/cpu/test.cc:101-144
    wte = torch.tensor([[0.1, 0.2], [0.3, 0.4], [0.2, 0.3], [0.4, 0.5], [0.7, 0.8]]).cuda()
    ids = torch.tensor([0, 1, 2, 1, 3, 4], dtype=torch.int32).cuda()
    want = torch.tensor([[0.1, 0.2], [0.3, 0.4], [0.2, 0.3], [0.3, 0.4], [0.4, 0.5], [0.7, 0.8]])
    assert torch.allclose(ops.embed(wte, ids, 1.0).cpu(), want)


# ------------------------------------------------------------------------------- norm
@pytest.mark.parametrize("dtype", DTYPES)
# 10/11: src/flint/cuda/test.cc:243-248; rows of up to 2,048, 4,096, 8,192 and 16,384 elements that are a
# multiple of 4 have a kernel form each, the others the plain one
@pytest.mark.parametrize("width", [10, 11, 192, 2050, 4096, 5120, 8192, 9000, 16384, 16388, 20002])
def test_add_rmsnorm(ops, dtype, width):
    m, eps = 7, 1e-5
    res = rnd((m, width), torch.float32, 2, 3.0).cuda()
    delta = rnd((m, width), dtype, 3).cuda()
    w = (1.0 + rnd((width,), torch.float32, 4, 0.3)).cuda()
    res0 = res.clone()
    out = ops.add_rmsnorm(res, delta, w, eps, dtype)
    x = res0.double() + delta.double()
    assert torch.allclose(res.double(), x, rtol=1e-6, atol=1e-6)          # the sum is kept in 32-bit
    ref = x * w.double() / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    assert close(out, ref, dtype)
    # no delta, gathered rows
    rows = torch.tensor([5, 0, 5], dtype=torch.int32).cuda()
    before = res.clone()
    out = ops.add_rmsnorm(res, None, w, eps, dtype, rows)
    assert torch.equal(res, before)
    assert close(out, ref[rows.long()], dtype)


@pytest.mark.parametrize("width", [2048, 5120, 8192, 12000])
@pytest.mark.parametrize("n_delta", [1, 3, 11])
def test_add_rmsnorm_of_several_matrices(ops, width, n_delta):
    """Several float32 matrices are added into the stream in their order, at every form of the kernel."""
    m = 5
    res = rnd((m, width), torch.float32, 5, 3.0).cuda()
    parts = rnd((n_delta, m, width), torch.float32, 6).cuda()
    w = (1.0 + rnd((width,), torch.float32, 7, 0.3)).cuda()
    want = res.clone()
    for j in range(n_delta):
        want += parts[j]
    out = ops.add_rmsnorm(res, parts, w, 1e-5, torch.bfloat16)
    assert torch.equal(res, want)
    x = want.double()
    assert close(out, x * w.double() / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5), torch.bfloat16)


def test_rmsnorm_zero_and_eps(ops):
    res = torch.zeros((2, 64), device="cuda")
    w = torch.ones(64, device="cuda")
    out = ops.add_rmsnorm(res, None, w, 1e-6, torch.float32)
    assert torch.equal(out.cpu(), torch.zeros(2, 64))                      # eps inside the root: no NaN
    res = torch.full((1, 64), 1e-3, device="cuda")
    out = ops.add_rmsnorm(res, None, w, 1e-2, torch.float32)                # eps dominates
    assert torch.allclose(out.cpu(), torch.full((1, 64), 1e-3 / math.sqrt(1e-6 + 1e-2)), rtol=1e-5)


# ------------------------------------------------------------------------------- matrix products
@pytest.mark.parametrize("mnk", [(1, 1, 1), (1, 513, 64), (7, 33, 129), (64, 64, 64), (65, 130, 257),
                                 (2, 1000, 192), (300, 70, 16), (1, 1, 2050)])
def test_gemm_f32(ops, mnk):
    m, n, k = mnk
    x = rnd((m, k), torch.float32, 5).cuda()
    w = rnd((n, k), torch.float32, 6).cuda()
    out = ops.linear(x, w, None, torch.float32)
    ref = x.double() @ w.double().t()
    assert max_err(out, ref) < 2e-6


@pytest.mark.parametrize("nk", [(1000, 2050), (37, 8200), (2048, 4096), (70, 17), (16, 64), (17, 65), (5, 3)])
def test_gemm_f32_of_few_rows_gives_the_same_bits(ops, nk):
    """Up to 16 rows go through a kernel of their own (16 rows of the weight a block, 64 elements
    of K between barriers, 16 bytes a load where K and the addresses allow): it adds the terms in
    the order of the kernel for many rows, so a row's bits do not depend on how many rows a step
    has.  K that is no multiple of 4, of 16 or of 64; weights of fewer than 16 rows; a view whose
    rows do not start at 16 bytes."""
    n, k = nk
    x = rnd((40, k), torch.float32, 15).cuda()
    w = rnd((n, k), torch.float32, 16).cuda()
    many = ops.linear(x, w, None, torch.float32)                 # 40 rows: the kernel for many rows
    assert max_err(many, x.double() @ w.double().t()) < 2e-6
    for m in (1, 7, 16):
        few = ops.linear(x[:m].contiguous(), w, None, torch.float32)
        assert torch.equal(few, many[:m])
    shifted = torch.cat([x.new_zeros(1), x[:3].reshape(-1)])[1:].view(3, k)     # rows that start 4 bytes off
    assert shifted.data_ptr() % 16 == 4 and torch.equal(ops.linear(shifted, w, None, torch.float32), many[:3])


def test_linear_bias_and_mixed_dtypes(ops):
    x = rnd((5, 40), torch.bfloat16, 7).cuda()
    w32 = rnd((24, 40), torch.float32, 8).cuda()        # a matrix stored in 32-bit stays so
    b = rnd((24,), torch.float32, 9).cuda()
    out = ops.linear(x, w32, b, torch.bfloat16)
    ref = x.double() @ w32.double().t() + b.double()
    assert out.dtype == torch.bfloat16 and close(out, ref, torch.bfloat16)


@pytest.mark.parametrize("m", [1, 3, 16, 17, 33, 64])
@pytest.mark.parametrize("nk", [(16, 8), (24, 136), (1000, 2048), (2050, 264), (40, 4104), (4112, 72)])
@pytest.mark.parametrize("out_dtype", DTYPES)
def test_gemm_skinny(ops, m, nk, out_dtype):
    n, k = nk
    x = rnd((m, k), torch.bfloat16, 10).cuda()
    w = rnd((n, k), torch.bfloat16, 11).cuda()
    out = ops.linear(x, w, None, out_dtype)
    assert out.dtype == out_dtype and tuple(out.shape) == (m, n)
    ref = x.double() @ w.double().t()
    assert max_err(out, ref) < (2e-6 if out_dtype == torch.float32 else BF16_2ULP)


def test_gemm_skinny_rows_per_block_and_batch_invariance(ops):
    k, n = 520, 300
    x = rnd((64, k), torch.bfloat16, 12).cuda()
    w = rnd((n, k), torch.bfloat16, 13).cuda()
    full = ops.linear(x, w, None, torch.float32)
    for m in (1, 5, 16, 40):                             # a row's result does not depend on the batch
        part = ops.linear(x[:m].contiguous(), w, None, torch.float32)
        assert torch.equal(part, full[:m])
    big = rnd((200, k), torch.bfloat16, 14).cuda()       # many rows with float32 output: chunks of 64
    out = ops.linear(big, w, None, torch.float32)
    assert max_err(out, big.double() @ w.double().t()) < 2e-6
    half = ops.linear(x, w, None, torch.bfloat16)         # the bfloat16 output is the rounded sum
    assert torch.equal(half, full.to(torch.bfloat16))


@pytest.mark.parametrize("m", [1, 7, 16, 30, 64])
@pytest.mark.parametrize("ik", [(16, 8), (48, 136), (160, 64), (512, 192), (8192, 2048), (208, 1032)])
def test_gemm_skinny_swiglu(ops, m, ik):
    inter, k = ik
    x = rnd((m, k), torch.bfloat16, 20).cuda()
    w = rnd((2 * inter, k), torch.bfloat16, 21, 3.0 / k ** 0.5).cuda()
    out = ops.linear_swiglu(x, w)
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (m, inter)
    gu = (x.double() @ w.double().t()).to(torch.bfloat16).double()    # the product is stored rounded
    g, u = gu[:, :inter], gu[:, inter:]
    ref = g / (1 + torch.exp(-g)) * u
    assert max_err(out, ref) < 2 * BF16_2ULP
    ops.fast_gemm = False                                               # the unfused path agrees
    try:
        slow = ops.linear_swiglu(x, w)
    finally:
        ops.fast_gemm = True
    assert max_err(slow, ref) < 2 * BF16_2ULP
    swapped = u / (1 + torch.exp(-u)) * g                               # gating the wrong half must differ
    assert max_err(out, swapped) > 0.05


def test_gemm_skinny_refuses(ops):
    x = rnd((2, 12), torch.bfloat16, 1).cuda()           # K not a multiple of 8: the library product runs
    w = rnd((16, 12), torch.bfloat16, 2).cuda()
    out = ops.linear(x, w, None, torch.bfloat16)
    assert close(out, x.double() @ w.double().t(), torch.bfloat16)
    c = torch.empty((2, 16), dtype=torch.bfloat16, device="cuda")
    st = ops.lib.llm_gemm_skinny_bf16(x.data_ptr(), w.data_ptr(), c.data_ptr(), 0, 1, 2, 16, 12, 12, 1, 0)
    assert st == 1                                        # refused, not wrong


@pytest.mark.parametrize("nk", [(16, 8), (300, 520), (2050, 264), (3072, 2048), (40, 4104), (4128, 136)])
def test_prepared_weight_gives_the_same_bits(ops, nk):
    """The copy tiled for the matrix cores holds the same numbers: every product for few rows
    returns the same bits from it as from the matrix, and the product for many rows reads the matrix."""
    from libllm_amd.hip.ops import PreparedWeight
    n, k = nk
    w = rnd((n, k), torch.bfloat16, 60).cuda()
    pw = ops.prepare_weight(w)
    assert isinstance(pw, PreparedWeight) and tuple(pw.shape) == (n, k)
    for m in (1, 9, 40, 130):
        x = rnd((m, k), torch.bfloat16, 61).cuda()
        for out_dtype in DTYPES:
            a, b = ops.linear(x, pw, None, out_dtype), ops.linear(x, w, None, out_dtype)
            if m > ops.SKINNY_ROWS and out_dtype == torch.float32:
                # float32 results of many rows: the product for 33 to 128 rows where there is a
                # tiled copy and K allows it, else the one for few rows in passes; both are right
                ref = x.double() @ w.double().t()
                assert close(a, ref, torch.float32) and close(b, ref, torch.float32)
            else:
                assert torch.equal(a, b)
    x = rnd((9, k), torch.bfloat16, 61).cuda()
    a, b = torch.ones((9, n), device="cuda"), torch.ones((9, n), device="cuda")
    ops.linear(x, pw, None, torch.bfloat16, residual=a)
    ops.linear(x, w, None, torch.bfloat16, residual=b)
    assert torch.equal(a, b)
    if n % 32 == 0:
        assert torch.equal(ops.linear_swiglu(x, pw), ops.linear_swiglu(x, w))
        head = w[:n // 2]                                   # the leading rows share the tiled copy
        ph = ops.prepare_weight(head, like=pw)
        assert ph.tiled is pw.tiled
        assert torch.equal(ops.linear(x, ph, None, torch.float32), ops.linear(x, head.contiguous(), None, torch.float32))
    stream = rnd((9, k), torch.float32, 62, 3.0).cuda()
    wn = (1.0 + 0.2 * rnd((k,), torch.float32, 63)).cuda()
    lazy = ops.normed(stream, wn, 1e-5)
    assert torch.equal(ops.linear(lazy, pw, None, torch.bfloat16), ops.linear(lazy, w, None, torch.bfloat16))
    w32 = rnd((24, 40), torch.float32, 64).cuda()
    assert ops.prepare_weight(w32) is w32                   # a 32-bit matrix is left as it is


def test_weight_rows_may_lie_apart(ops):
    """A weight that is a view of some columns of a wider matrix: the same bits from every product."""
    w = rnd((300, 1024), torch.bfloat16, 50).cuda()
    wide = torch.zeros((300, 1024 + 64), dtype=torch.bfloat16, device="cuda")
    wide[:, :1024] = w
    ws = wide[:, :1024]
    assert ws.stride(0) == 1088 and torch.equal(ws, w)
    res0 = rnd((9, 300), torch.float32, 53).cuda()
    for m in (1, 9, 64, 200):                             # skinny and library products
        x = rnd((m, 1024), torch.bfloat16, 52).cuda()
        for out_dtype in DTYPES:
            assert torch.equal(ops.linear(x, ws, None, out_dtype), ops.linear(x, w, None, out_dtype))
    x = rnd((9, 1024), torch.bfloat16, 52).cuda()
    a, b = res0.clone(), res0.clone()
    ops.linear(x, ws, None, torch.bfloat16, residual=a)
    ops.linear(x, w, None, torch.bfloat16, residual=b)
    assert torch.equal(a, b)
    w2 = rnd((320, 1024), torch.bfloat16, 54).cuda()
    wide2 = torch.zeros((320, 1032), dtype=torch.bfloat16, device="cuda")
    wide2[:, :1024] = w2
    assert torch.equal(ops.linear_swiglu(x, wide2[:, :1024]), ops.linear_swiglu(x, w2))


@pytest.mark.parametrize("m", [1, 5, 16, 32, 40])
@pytest.mark.parametrize("nk", [(16, 8), (300, 520), (2048, 2048), (72, 4104)])
def test_gemm_skinny_adds_into_the_stream(ops, monkeypatch, m, nk):
    """Up to ``ACCUM_ROWS`` rows the product adds into the stream itself and returns None; beyond,
    the product is returned (a matrix, or slices over K) for the norm to add and the stream is left alone.  Forced to 64
    the kernel adds for 40 rows too."""
    n, k = nk
    x = rnd((m, k), torch.bfloat16, 30).cuda()
    w = rnd((n, k), torch.bfloat16, 31).cuda()
    ref = x.double() @ w.double().t()
    for limit in (ops.ACCUM_ROWS, 64):
        monkeypatch.setattr(ops, "ACCUM_ROWS", limit)
        res = rnd((m, n), torch.float32, 32, 5.0).cuda()
        before = res.clone()
        out = ops.linear(x, w, None, torch.bfloat16, residual=res)
        if m > limit:                       # the product comes back, whole or in slices of K, for the norm to add
            assert out is not None and torch.equal(res, before)
            assert close(out.sum(0) if out.dim() == 3 else out, ref, torch.bfloat16)
            continue
        assert out is None
        assert max_err(res, before.double() + ref.cuda()) < 2e-6
        plain = ops.linear(x, w, None, torch.float32)          # the same sums as the plain product
        assert torch.equal(res, before + plain)


@pytest.mark.parametrize("m", [1, 3, 8, 16, 20])
@pytest.mark.parametrize("nk", [(16, 8), (300, 520), (3072, 2048), (72, 1032)])
@pytest.mark.parametrize("gather", [False, True])
def test_products_of_rows_still_to_be_normalised(ops, m, nk, gather):
    """A product over a ``normed`` record: the norm kernel runs on just those rows, then the
    product.  Against the plain formulas, and against the two steps called one by one."""
    n, k = nk
    stream = rnd((m + 3, k), torch.float32, 33, 7.0).cuda()
    stream[0] *= 1e-3                                      # rows of very different size
    wn = (1.0 + 0.3 * rnd((k,), torch.float32, 34)).cuda()
    w = rnd((n, k), torch.bfloat16, 35).cuda()
    rows = torch.tensor([(3 * i + 1) % (m + 3) for i in range(m)], dtype=torch.int32, device="cuda") if gather else None
    src = stream[rows.long()] if gather else stream[:m]
    sd = src.double()
    h = sd * wn.double() / torch.sqrt((sd * sd).mean(dim=-1, keepdim=True) + 1e-5)
    ref = h @ w.double().t()
    lazy = ops.normed(stream if gather else stream[:m].contiguous(), wn, 1e-5, rows)
    for out_dtype in DTYPES:
        out = ops.linear(lazy, w, None, out_dtype)
        assert out.dtype == out_dtype and tuple(out.shape) == (m, n)
        assert max_err(out, ref) < (BF16_2ULP if out_dtype == torch.bfloat16 else 2.0 ** -8)
    hb = ops.add_rmsnorm(stream if gather else stream[:m].contiguous(), None, wn, 1e-5, torch.bfloat16, rows)
    unfused = ops.linear(hb, w, None, torch.float32)
    assert max_err(ops.linear(lazy, w, None, torch.float32), unfused) < 2.0 ** -7
    if n % 32 == 0:
        g, u = ref[:, :n // 2], ref[:, n // 2:]
        sw = ops.linear_swiglu(lazy, w, torch.bfloat16)
        assert max_err(sw, g / (1 + torch.exp(-g)) * u) < 4 * BF16_2ULP


@pytest.mark.parametrize("m", [1, 3, 8, 16])
@pytest.mark.parametrize("nk", [(16, 8), (304, 520), (2048, 2048), (2048, 8192), (4096, 1032)])
def test_product_prepares_the_norm_that_follows(ops, m, nk):
    """A product that adds into the stream, told which RMS norm reads the stream next: the stream
    gets the same bits as without, ``raw`` is the new stream times the norm's weight rounded once,
    ``ssq`` holds the sums of squares over tiles of 16 columns; a row's values do not depend on
    the other rows of the step."""
    n, k = nk
    x = rnd((m, k), torch.bfloat16, 90).cuda()
    w = rnd((n, k), torch.bfloat16, 91).cuda()
    pw = ops.prepare_weight(w)
    nw = (1.0 + 0.3 * rnd((n,), torch.float32, 92)).cuda()
    res = rnd((m, n), torch.float32, 93, 5.0).cuda()
    res[0] *= 1e-3
    plain = res.clone()
    assert ops.linear(x, pw, None, torch.bfloat16, residual=plain) is None
    pre = ops.linear(x, pw, None, torch.bfloat16, residual=res, then_norm=(nw, 1e-5))
    assert pre is not None and pre.weight is nw and pre.eps == 1e-5
    assert torch.equal(res, plain)
    assert torch.equal(pre.raw, (res * nw).to(torch.bfloat16))
    want = (res.double() ** 2).reshape(m, n // 16, 16).sum(-1)
    assert tuple(pre.ssq.shape) == (m, n // 16) and max_err(pre.ssq, want) < 1e-6
    one = rnd((m, n), torch.float32, 93, 5.0).cuda()
    one[0] *= 1e-3
    one = one[m - 1:].contiguous()
    alone = ops.linear(x[m - 1:].contiguous(), pw, None, torch.bfloat16, residual=one, then_norm=(nw, 1e-5))
    assert torch.equal(alone.raw[0], pre.raw[m - 1]) and torch.equal(alone.ssq[0], pre.ssq[m - 1])
    # more rows than the product adds for, or a width that is no multiple of 16: no record
    if m == 16:
        big = rnd((17, n), torch.float32, 94).cuda()
        out = ops.linear(rnd((17, k), torch.bfloat16, 95).cuda(), pw, None, torch.bfloat16, residual=big,
                         then_norm=(nw, 1e-5))
        assert out is None or isinstance(out, torch.Tensor)


@pytest.mark.parametrize("m", [1, 5, 16])
@pytest.mark.parametrize("width,n", [(2048, 3072), (2048, 16384), (528, 304), (4096, 1024)])
def test_products_over_a_prepared_norm(ops, m, width, n):
    """The product after a prepared norm takes ``raw`` as its rows and multiplies its sums by the
    row's rsqrt(mean(x^2) + eps): plain product, SwiGLU and the rotary q|k|v product, against the
    plain formulas in float64 and against the norm kernel followed by the same product."""
    kin = 256
    x = rnd((m, kin), torch.bfloat16, 96).cuda()
    wo = ops.prepare_weight(rnd((width, kin), torch.bfloat16, 97, 0.5).cuda())
    nw = (1.0 + 0.3 * rnd((width,), torch.float32, 98)).cuda()
    res = rnd((m, width), torch.float32, 99, 4.0).cuda()
    res[0] *= 1e-3
    eps = 1e-5
    pre = ops.linear(x, wo, None, torch.bfloat16, residual=res, then_norm=(nw, eps))
    lazy = ops.normed(res, nw, eps, pre=pre)
    assert lazy.pre is pre
    assert ops.normed(res, nw, 1e-6, pre=pre).pre is None                 # another norm than the one prepared
    assert ops.normed(res, nw.clone(), eps, pre=pre).pre is None
    assert ops.normed(res, nw, eps, torch.arange(m, dtype=torch.int32, device="cuda"), pre=pre).pre is None
    w = rnd((n, width), torch.bfloat16, 100).cuda()
    pw = ops.prepare_weight(w)
    rd = res.double()
    h = rd * nw.double() / torch.sqrt((rd * rd).mean(-1, keepdim=True) + eps)
    ref = h @ w.double().t()
    hb = ops.add_rmsnorm(res, None, nw, eps, torch.bfloat16)              # the norm kernel's rows
    for out_dtype in DTYPES:
        out = ops.linear(lazy, pw, None, out_dtype)
        assert out.dtype == out_dtype and max_err(out, ref) < (BF16_2ULP if out_dtype == torch.bfloat16 else 2.0 ** -8)
    assert max_err(ops.linear(lazy, pw, None, torch.float32), ops.linear(hb, pw, None, torch.float32)) < 2.0 ** -7
    if n % 32 == 0:
        g, u = ref[:, :n // 2], ref[:, n // 2:]
        sw = ops.linear_swiglu(lazy, pw, torch.bfloat16)
        assert max_err(sw, g / (1 + torch.exp(-g)) * u) < 4 * BF16_2ULP
        assert max_err(sw, ops.linear_swiglu(hb, pw)) < 4 * BF16_2ULP
    # the rotary product: the same queries and cache as from the norm kernel's rows, up to rounding
    hd = 64
    if n % hd == 0 and n // hd >= 3:
        n_kv = max(1, n // hd // 6)
        n_heads = n // hd - 2 * n_kv
        seqs = [(i, 3 * i, 1) for i in range(m)]
        ctx = make_ctx(ops, torch.bfloat16, seqs)
        cos = torch.cos(rnd((64, hd // 2), torch.float32, 101)).cuda()
        sin = torch.sin(rnd((64, hd // 2), torch.float32, 101)).cuda()
        outs = []
        for rows in (lazy, hb):
            kv = make_kv("cuda", torch.bfloat16, m, 1, n_kv, hd, seed=1)
            q = ops.qkv_rope(rows, pw, None, n_heads, n_kv, hd, cos, sin, hd, ctx, kv, True, True, torch.bfloat16)
            outs.append((q[:, :n_heads * hd].clone(), kv.plane("k").clone(), kv.plane("v").clone()))
        for a, b in zip(*outs):
            assert max_err(a, b) < BF16_2ULP
        assert float(outs[0][1].float().abs().max()) > 0


@pytest.mark.parametrize("m", [17, 33, 40, 64])
@pytest.mark.parametrize("nk", [(128, 2048), (2048, 2048), (2048, 8192), (3072, 3072), (200, 1536)])
def test_products_in_slices_of_k(ops, monkeypatch, m, nk):
    """From 17 to 64 rows a product that adds into the stream is computed over slices of K, each
    slice to a float32 matrix of its own, and the norm kernel that follows adds them in order:
    against the plain formulas, from the weight as it lies and from its tiled copy (the same
    bits), and the same bits when other rows share the step.  (From 33 rows on the product for 33
    to 128 rows takes the weights it can, see below; here it is switched off.)"""
    n, k = nk
    monkeypatch.setattr(ops, "ACCUM_ROWS", 16)               # so that 17 rows take this path too
    monkeypatch.setattr(ops, "MID_FROM", 65)
    ks = ops._k_split(n, k)
    assert ks > 1 and k % (ks * 32) == 0
    x = rnd((m, k), torch.bfloat16, 80).cuda()
    w = rnd((n, k), torch.bfloat16, 81).cuda()
    pw = ops.prepare_weight(w)
    res = rnd((m, n), torch.float32, 82, 3.0).cuda()
    parts = ops.linear(x, pw, None, torch.bfloat16, residual=res)
    assert tuple(parts.shape) == (ks, m, n) and parts.dtype == torch.float32
    ref = x.double() @ w.double().t()
    assert max_err(parts.double().sum(0), ref.cuda()) < 2e-6
    for j in range(ks):                                      # every slice is the product over its part of K
        sl = slice(j * (k // ks), (j + 1) * (k // ks))
        assert max_err(parts[j], (x[:, sl].double() @ w[:, sl].double().t()).cuda()) < 2e-6
    plain = torch.empty_like(parts)
    ops._skinny(x, w, plain, ops._EPI_NONE, 0, m, k_split=ks)
    assert torch.equal(plain, parts)
    fewer = ops.linear(x[:17].contiguous(), pw, None, torch.bfloat16, residual=res[:17].contiguous())
    assert torch.equal(fewer, parts[:, :17])                 # a row's sums do not depend on the other rows
    # the norm adds the slices into the stream in their order and normalises
    wn = (1.0 + 0.2 * rnd((n,), torch.float32, 83)).cuda()
    stream = res.clone()
    out = ops.add_rmsnorm(stream, parts, wn, 1e-5, torch.bfloat16)
    want = res.clone()
    for j in range(ks):
        want += parts[j]
    assert torch.equal(stream, want)
    sd = want.double()
    assert close(out, sd * wn.double() / torch.sqrt((sd * sd).mean(-1, keepdim=True) + 1e-5), torch.bfloat16)
    # a buffer for the slices that is too small, or slices that do not divide K, are refused
    from libllm_amd.errors import KernelError
    with pytest.raises(KernelError):
        ops._skinny(x, w, plain, ops._EPI_NONE, 0, m, k_split=7)


# ---------------------------------------------------------------- the product for 33 to 128 rows
@pytest.mark.parametrize("m", [33, 48, 50, 64, 65, 80, 97, 128])
@pytest.mark.parametrize("nk", [(64, 128), (48, 256), (1000, 640), (3072, 3072), (2048, 8192)])
def test_gemm_mid(ops, m, nk):
    """Plain as bfloat16, and in slices of K as float32 matrices, against float64; weights whose
    rows are no multiple of 64 or of 16, one chunk of K and many."""
    n, k = nk
    x = rnd((m, k), torch.bfloat16, 3).cuda()
    w = ops.prepare_weight(rnd((n, k), torch.bfloat16, 4, scale=0.05).cuda())
    ref = x.double() @ w.w.double().t()
    out = ops._mid(x, w, torch.empty((m, n), dtype=torch.bfloat16, device="cuda"), ops._EPI_NONE)
    assert close(out, ref, torch.bfloat16)
    for ks in sorted({1, 2 if (k // 128) % 2 == 0 else 1, k // 128}):
        parts = ops._mid(x, w, torch.empty((ks, m, n), dtype=torch.float32, device="cuda"), ops._EPI_NONE, ks)
        total = parts[0].clone()
        for j in range(1, ks):
            total += parts[j]
        assert close(total, ref, torch.float32)


@pytest.mark.parametrize("m", [34, 64, 66, 128])
@pytest.mark.parametrize("ik", [(32, 128), (208, 384), (8192, 2048)])
def test_gemm_mid_swiglu(ops, m, ik):
    """silu(gate) * up over a stacked weight, gate and up rounded to bfloat16 first as the
    unfused path stores them: the same bits as the library's product and the SiLU-mul kernel
    give wherever the two products agree on every rounded gate and up, close everywhere."""
    inter, k = ik
    x = rnd((m, k), torch.bfloat16, 5).cuda()
    w = ops.prepare_weight(rnd((2 * inter, k), torch.bfloat16, 6, scale=0.05).cuda())
    out = ops._mid(x, w, torch.empty((m, inter), dtype=torch.bfloat16, device="cuda"), ops._EPI_SWIGLU)
    gu = (x.double() @ w.w.double().t()).bfloat16().double()
    g, u = gu[:, :inter], gu[:, inter:]
    ref = u * g / (1 + torch.exp(-g))
    err = ((out.double() - ref).abs() / (ref.abs() + ref.abs().mean())).max().item()
    assert err < 0.02, err


def test_gemm_mid_rows_do_not_depend_on_the_batch(ops):
    """A row's sums are added along K by the same two waves in the same order whatever the other
    rows are: the same bits at 33, 48, 65, 100 and 128 rows, and with the row at another place."""
    n, k = 1024, 1024
    x = rnd((128, k), torch.bfloat16, 7).cuda()
    w = ops.prepare_weight(rnd((n, k), torch.bfloat16, 8, scale=0.05).cuda())
    full = ops._mid(x, w, torch.empty((128, n), dtype=torch.bfloat16, device="cuda"), ops._EPI_NONE)
    for m in (33, 48, 64, 65, 100):
        part = ops._mid(x[:m].contiguous(), w, torch.empty((m, n), dtype=torch.bfloat16, device="cuda"), ops._EPI_NONE)
        assert torch.equal(part, full[:m])
    moved = torch.cat([x[64:], x[:64]]).contiguous()
    out = ops._mid(moved, w, torch.empty((128, n), dtype=torch.bfloat16, device="cuda"), ops._EPI_NONE)
    assert torch.equal(out[:64], full[64:]) and torch.equal(out[64:], full[:64])


def test_steps_of_33_to_64_rows_use_it_where_it_fills_the_device(ops):
    """A product that adds into the stream goes to it if its slices of K give blocks enough, else to
    the product for few rows; the gate and up product always; a row's bits are the same at 33, 48 and
    64 rows."""
    x = rnd((64, 8192), torch.bfloat16, 11).cuda()
    down = ops.prepare_weight(rnd((2048, 8192), torch.bfloat16, 12, scale=0.05).cuda())
    small = ops.prepare_weight(rnd((2048, 2048), torch.bfloat16, 13, scale=0.05).cuda())
    gate_up = ops.prepare_weight(rnd((2 * 4096, 2048), torch.bfloat16, 14, scale=0.05).cuda())
    res = torch.zeros((64, 2048), dtype=torch.float32, device="cuda")
    ks = ops._k_split_mid(2048, 8192)
    assert ks * 32 >= ops.MID_FILL * ops.units
    whole = None
    for m in (64, 48, 33):
        parts = ops.linear(x[:m].contiguous(), down, None, torch.bfloat16, residual=res[:m].contiguous())
        assert tuple(parts.shape) == (ks, m, 2048)
        assert torch.equal(parts, ops._mid(x[:m].contiguous(), down, torch.empty_like(parts), ops._EPI_NONE, ks))
        whole = parts if whole is None else whole
        assert torch.equal(parts, whole[:, :m])
    xs = x[:, :2048].contiguous()
    few = ops.linear(xs, small, None, torch.bfloat16, residual=res)
    ks_few = ops._k_split(2048, 2048)
    assert ops._k_split_mid(2048, 2048) * 32 < ops.MID_FILL * ops.units and tuple(few.shape) == (ks_few, 64, 2048)
    plain = torch.empty_like(few)
    ops._skinny(xs, small, plain, ops._EPI_NONE, 0, 64, k_split=ks_few)
    assert torch.equal(few, plain)
    act = ops.linear_swiglu(xs, gate_up)
    assert torch.equal(act, ops._mid(xs, gate_up, torch.empty_like(act), ops._EPI_SWIGLU))
    assert torch.equal(ops.linear_swiglu(xs[:40].contiguous(), gate_up), act[:40])


def test_steps_of_129_to_256_rows_take_it_by_the_product(ops):
    """Which products of a step of 129 to 256 rows go to the product for 33 to 128 rows in two
    slabs, and which stay with the library or the product for many rows: by the weight's shape,
    as measured (the down and output products in slices of K, half as many as up to 128 rows;
    q|k|v where its blocks fill most of one round of the units; gate|up where all its blocks run
    at once).  Every result against float64."""
    took = []
    real_mid, real_lib, real_wide = ops._mid, ops._library_product, ops._wide
    ops._mid = lambda *a, **kw: took.append(("mid", a[4] if len(a) > 4 else kw.get("k_split", 1))) or real_mid(*a, **kw)
    ops._library_product = lambda *a, **kw: took.append(("library", 1)) or real_lib(*a, **kw)
    ops._wide = lambda *a, **kw: took.append(("wide", 1)) or real_wide(*a, **kw)
    try:
        m = 200
        for what, (n, k), adds, want in (("down 1B", (2048, 8192), True, ("mid", 4)), ("down 8B", (4096, 14336), True, ("mid", 2)),
                                         ("q|k|v 1B", (3072, 2048), False, ("library", 1)), ("q|k|v 3B", (5120, 3072), False, ("mid", 1)),
                                         ("q|k|v 8B", (6144, 4096), False, ("mid", 1)), ("q|k|v wide", (10240, 8192), False, ("library", 1))):
            x = rnd((m, k), torch.bfloat16, 41).cuda()
            w = ops.prepare_weight(rnd((n, k), torch.bfloat16, 42, scale=0.02).cuda())
            res = torch.zeros((m, n), dtype=torch.float32, device="cuda")
            del took[:]
            out = ops.linear(x, w, None, torch.bfloat16, residual=res if adds else None)
            assert took == [want], (what, took)
            ref = x.double() @ w.w.double().t()
            if adds:
                assert tuple(out.shape) == (want[1], m, n) and close(out.sum(0), ref, torch.float32, f32=3e-5)
            else:
                assert close(out, ref, torch.bfloat16)
        for what, (inter, k), want in (("gate|up 1B", (8192, 2048), "mid"), ("gate|up 8B", (14336, 4096), "library")):      # (at 256 rows the product for many rows, whose tiles it then fills)
            x = rnd((m, k), torch.bfloat16, 43).cuda()
            w = ops.prepare_weight(rnd((2 * inter, k), torch.bfloat16, 44, scale=0.02).cuda())
            del took[:]
            out = ops.linear_swiglu(x, w)
            assert [t[0] for t in took] == [want], (what, took)
            gu = (x.double() @ w.w.double().t()).bfloat16().double()
            ref = gu[:, inter:] * gu[:, :inter] / (1 + torch.exp(-gu[:, :inter]))
            assert ((out.double() - ref).abs() / (ref.abs() + ref.abs().mean())).max().item() < 0.02
    finally:
        ops._mid, ops._library_product, ops._wide = real_mid, real_lib, real_wide


def test_logits_of_65_to_128_rows_take_one_pass(ops):
    """Float32 results without a stream to add to (the head) go through the product for 33 to 128
    rows from 65 rows on, where the product for few rows would read the weight twice; a normed
    record is made into rows first."""
    x = rnd((100, 256), torch.bfloat16, 21).cuda()
    w = ops.prepare_weight(rnd((1000, 256), torch.bfloat16, 22, scale=0.05).cuda())
    out = ops.linear(x, w, None, torch.float32)
    assert out.dtype == torch.float32 and tuple(out.shape) == (100, 1000)
    assert torch.equal(out, ops._mid(x, w, torch.empty((1, 100, 1000), dtype=torch.float32, device="cuda"), ops._EPI_NONE, 1)[0])
    assert close(out, x.double() @ w.w.double().t(), torch.float32)
    few = ops.linear(x[:64].contiguous(), w, None, torch.float32)            # up to 64 rows: the product for few rows
    assert max_err(few, out[:64]) < 2e-6
    res = rnd((100, 256), torch.float32, 23, 2.0).cuda()
    wn = (1.0 + 0.1 * rnd((256,), torch.float32, 24)).cuda()
    lazy = ops.normed(res, wn, 1e-5)
    rows = ops.add_rmsnorm(res, None, wn, 1e-5, torch.bfloat16)
    assert torch.equal(ops.linear(lazy, w, None, torch.float32), ops.linear(rows, w, None, torch.float32))


@pytest.mark.parametrize("n", [1000, 517])
def test_float32_results_of_many_rows_in_passes(ops, n):
    """Logits (float32, no residual) of 65 rows and more go through the product for 33 to 256
    rows, in one pass up to 256 rows and in even passes beyond; a row's bits do not depend on
    how many rows there are, nor on the pass it falls into.  A vocabulary that is no multiple of
    4 has rows that are not 16 bytes apart: every pass still starts at an aligned row."""
    k = 256
    x = rnd((1100, k), torch.bfloat16, 21).cuda()
    w = ops.prepare_weight(rnd((n, k), torch.bfloat16, 22, scale=0.05).cuda())
    ref = x.double() @ w.w.double().t()
    calls = []
    real = ops._mid
    ops._mid = lambda *a, **kw: calls.append(a[0].shape[0]) or real(*a, **kw)
    try:
        full = ops.linear(x, w, None, torch.float32)
        top = ops._mid_rows()                                 # most rows of a pass: 256, in two slabs beyond 128
        assert sum(calls) == 1100 and len(calls) == -(-1100 // top) and all(49 <= c <= top for c in calls)
        assert full.dtype == torch.float32 and close(full, ref, torch.float32)
        for m in (65, 128, 129, 255, 257, 1000):
            del calls[:]
            part = ops.linear(x[:m], w, None, torch.float32)
            assert sum(calls) == m and len(calls) == -(-m // top)
            assert torch.equal(part, full[:m])
    finally:
        ops._mid = real


@pytest.mark.parametrize("m", [129, 130, 160, 161, 200, 255, 256])
@pytest.mark.parametrize("nk", [(64, 128), (1000, 256), (2048, 2048), (520, 1024), (4, 128)])
def test_gemm_mid_in_two_slabs(ops, m, nk):
    """129 to 256 rows go in two slabs of rows, a block each for every tile of W: plain as
    bfloat16, in slices of K as float32 matrices, and gated, against float64; a row's bits are
    those of the same row among up to 128 (the slabs split at other rows than the passes do);
    weights whose tiles are no multiple of 8 (the grid is rounded up to whole rounds of the
    chiplets), a sentinel behind the result."""
    n, k = nk
    x = rnd((m, k), torch.bfloat16, 31).cuda()
    w = ops.prepare_weight(rnd((n, k), torch.bfloat16, 32, scale=0.05).cuda())
    ref = x.double() @ w.w.double().t()
    buf = torch.full((m * n + 64,), 7.0, dtype=torch.bfloat16, device="cuda")
    out = ops._mid(x, w, buf[:m * n].view(m, n), ops._EPI_NONE)
    assert close(out, ref, torch.bfloat16) and (buf[m * n:] == 7.0).all()
    first = ops._mid(x[:128], w, torch.empty((128, n), dtype=torch.bfloat16, device="cuda"), ops._EPI_NONE)
    rest = ops._mid(x[m - 100:], w, torch.empty((100, n), dtype=torch.bfloat16, device="cuda"), ops._EPI_NONE)
    assert torch.equal(out[:128], first) and torch.equal(out[m - 100:], rest)
    ks = 2 if (k // 128) % 2 == 0 else 1
    parts = ops._mid(x, w, torch.empty((ks, m, n), dtype=torch.float32, device="cuda"), ops._EPI_NONE, ks)
    total = parts[0].clone()
    for j in range(1, ks):
        total += parts[j]
    assert close(total, ref, torch.float32)
    if n % 32 == 0:
        inter = n // 2
        got = ops._mid(x, w, torch.empty((m, inter), dtype=torch.bfloat16, device="cuda"), ops._EPI_SWIGLU)
        one = torch.cat([ops._mid(x[:128], w, torch.empty((128, inter), dtype=torch.bfloat16, device="cuda"), ops._EPI_SWIGLU),
                         ops._mid(x[128:] if m - 128 >= 33 else x[m - 33:], w,
                                  torch.empty((max(m - 128, 33), inter), dtype=torch.bfloat16, device="cuda"), ops._EPI_SWIGLU)[-(m - 128):]])
        assert torch.equal(got, one)


def test_gemm_mid_refuses(ops):
    from libllm_amd.errors import KernelError
    w = ops.prepare_weight(rnd((64, 256), torch.bfloat16, 1).cuda())
    x = rnd((128, 256), torch.bfloat16, 2).cuda()
    for rows, ks in ((32, 1), (257, 1), (100, 3)):                     # too few rows, too many, slices that do not divide K
        with pytest.raises(KernelError):
            xs = torch.cat([x, x, x])[:rows].contiguous()
            ops._mid(xs, w, torch.empty((ks, rows, 64), dtype=torch.float32, device="cuda"), ops._EPI_NONE, ks)
    w2 = ops.prepare_weight(rnd((64, 200), torch.bfloat16, 1).cuda())    # K no multiple of the chunk
    assert not ops._mid_ok(rnd((100, 200), torch.bfloat16, 2).cuda(), w2, 100, 200)
    with pytest.raises(KernelError):
        ops._mid(rnd((100, 200), torch.bfloat16, 2).cuda(), w2, torch.empty((100, 64), dtype=torch.bfloat16, device="cuda"), ops._EPI_NONE)


# ---------------------------------------------------------------- other activations of the gate
def gate_act(name, g):
    """The gate's activation in float64: SiLU (src/flint/cuda/swiglu.cu:44-49), GELU in its tanh
    form, ReLU."""
    if name == "silu":
        return g / (1 + torch.exp(-g))
    if name == "relu":
        return torch.relu(g)
    return 0.5 * g * (1 + torch.tanh(math.sqrt(2 / math.pi) * (g + 0.044715 * g ** 3)))


@pytest.mark.parametrize("activation", ["gelu_tanh", "relu", "silu"])
def test_gated_products_with_other_activations(ops, activation):
    """act(gate) * up with another activation than SiLU, through every kernel that gates: the
    product for few rows (1, 16, 40 rows), the one for 33 to 128 rows, the one for many rows in
    both sizes of block, and the gating kernel behind the library's product, in both dtypes."""
    inter, k = 512, 256
    w = rnd((2 * inter, k), torch.bfloat16, 6, scale=0.08).cuda()
    pw = ops.prepare_weight(w)

    def want(x):
        gu = (x.double() @ w.double().t()).bfloat16().double()
        return gu[:, inter:] * gate_act(activation, gu[:, :inter])

    def err(out, ref):
        return ((out.double().cpu() - ref.cpu()).abs() / (ref.cpu().abs() + ref.cpu().abs().mean())).max().item()
    code = ops._EPI_SWIGLU | (ops.ACTIVATIONS[activation] << 4)
    for m in (1, 16, 40, 64):
        x = rnd((m, k), torch.bfloat16, m).cuda()
        out = torch.empty((m, inter), dtype=torch.bfloat16, device="cuda")
        ops._skinny(x, pw, out, code, 0, m)
        assert err(out, want(x)) < 0.02, ("few rows", m)
    for m in (33, 128):
        x = rnd((m, k), torch.bfloat16, m).cuda()
        out = ops._mid(x, pw, torch.empty((m, inter), dtype=torch.bfloat16, device="cuda"), code)
        assert err(out, want(x)) < 0.02, ("33 to 128 rows", m)
    for block_rows in (256, 128):
        x = rnd((300, k), torch.bfloat16, 9).cuda()
        out = ops._wide(x, pw, torch.empty((300, inter), dtype=torch.bfloat16, device="cuda"), code, block_rows)
        assert err(out, want(x)) < 0.02, ("many rows", block_rows)
    for m in (5, 200):                                            # whatever form the launcher picks
        x = rnd((m, k), torch.bfloat16, m + 1).cuda()
        assert err(ops.linear_swiglu(x, pw, torch.bfloat16, activation), want(x)) < 0.02
    for dtype in DTYPES:
        gu = rnd((9, 152), dtype, 15, 2.0).cuda()
        ref = gu[:, 76:].double() * gate_act(activation, gu[:, :76].double())
        assert close(ops.silu_mul(gu, activation), ref, dtype, f32=2e-6)
    gu = rnd((70, 1024), torch.bfloat16, 16, 2.0).cuda()        # the vector form
    assert close(ops.silu_mul(gu, activation), gu[:, 512:].double() * gate_act(activation, gu[:, :512].double()), torch.bfloat16)
    from libllm_amd.errors import KernelError
    with pytest.raises(KernelError, match="unknown activation"):
        ops.silu_mul(gu, "swish9")


# ---------------------------------------------------------------- the product for many rows
@pytest.mark.parametrize("block_rows", [256, 128])
@pytest.mark.parametrize("mnk", [(129, 64, 64), (300, 520, 128), (2048, 512, 256), (257, 1000, 192), (600, 264, 4096), (260, 384, 5120),
                                 (300, 268, 128), (129, 100, 64), (513, 4, 64)])
def test_gemm_wide(ops, mnk, block_rows):
    """Plain, against float64, both sizes of block: rows and weight rows that are no multiples of
    the tile, one tile of K and many, and weights whose number of rows is a multiple of 4 and not
    of 8 (268, 100, 4: every store is then of single elements, and the last lanes of a row store
    four).  The output lies inside a larger buffer of sentinels: nothing is written past it."""
    m, n, k = mnk
    x = rnd((m, k), torch.bfloat16, 3).cuda()
    w = rnd((n, k), torch.bfloat16, 4, scale=0.05).cuda()
    buf = torch.full((m * n + 64,), 7.0, dtype=torch.bfloat16, device="cuda")
    out = ops._wide(x, w, buf[:m * n].view(m, n), ops._EPI_NONE, block_rows)
    assert close(out, x.double() @ w.double().t(), torch.bfloat16)
    assert (buf[m * n:] == 7.0).all()
    # rows of X that lie apart, a prepared weight
    wide_x = torch.cat([x, x], dim=1)[:, :k]
    assert wide_x.stride(0) == 2 * k
    again = ops._wide(wide_x, ops.prepare_weight(w), torch.empty((m, n), dtype=torch.bfloat16, device="cuda"), ops._EPI_NONE, block_rows)
    assert torch.equal(again, out)


@pytest.mark.parametrize("block_rows", [256, 128])
@pytest.mark.parametrize("mik", [(257, 512, 192), (1000, 208, 64), (130, 16, 128), (2048, 8192, 2048)])
def test_gemm_wide_swiglu(ops, mik, block_rows):
    """silu(gate) * up over a stacked weight, gate and up rounded to bfloat16 first as the unfused
    path stores them; outputs that are no multiple of the tile."""
    m, inter, k = mik
    x = rnd((m, k), torch.bfloat16, 5).cuda()
    w = rnd((2 * inter, k), torch.bfloat16, 6, scale=0.05).cuda()
    out = ops._wide(x, w, torch.empty((m, inter), dtype=torch.bfloat16, device="cuda"), ops._EPI_SWIGLU, block_rows)
    gu = (x.double() @ w.double().t()).bfloat16().double()
    g, u = gu[:, :inter], gu[:, inter:]
    ref = u * g / (1 + torch.exp(-g))
    err = ((out.double() - ref).abs() / (ref.abs() + ref.abs().mean())).max().item()
    assert err < 0.02, err
    # a row's bits do not depend on the other rows of the step, nor on the size of block
    fewer = ops._wide(x[:129].contiguous(), w, torch.empty((129, inter), dtype=torch.bfloat16, device="cuda"), ops._EPI_SWIGLU, block_rows)
    assert torch.equal(fewer, out[:129])
    other = ops._wide(x, w, torch.empty((m, inter), dtype=torch.bfloat16, device="cuda"), ops._EPI_SWIGLU, 384 - block_rows)
    assert torch.equal(other, out)


def test_gemm_wide_is_used_where_its_tiles_fill_the_device(ops, monkeypatch):
    """The gate/up product of a prompt step goes to it by the rule of its launcher, and the result
    is what the kernel gives; elsewhere the library's product and the SiLU-mul kernel run."""
    from libllm_amd.errors import KernelError
    calls = []
    real = ops._wide
    monkeypatch.setattr(ops, "_wide", lambda *a: (calls.append(a[0].shape[0]), real(*a))[1])
    w = ops.prepare_weight(rnd((2 * 8192, 256), torch.bfloat16, 6, scale=0.05).cuda())
    sizes = []
    monkeypatch.setattr(ops, "_wide", lambda *a: (calls.append(a[0].shape[0]), sizes.append(a[4]), real(*a))[2])
    for m, used in ((1024, 256), (2048, 256), (768, 256), (512, 128), (384, 128), (520, 0), (700, 0), (200, 0), (128, 0)):
        x = rnd((m, 256), torch.bfloat16, m).cuda()
        calls.clear(), sizes.clear()
        out = ops.linear_swiglu(x, w)
        assert (sizes[0] if calls else 0) == used and ops._wide_ok(x, w, m, 256, 8192) == used, (m, calls, sizes)
        gu = (x.double() @ w.w.double().t()).bfloat16().double()
        ref = gu[:, 8192:] * gu[:, :8192] / (1 + torch.exp(-gu[:, :8192]))
        err = ((out.double() - ref).abs() / (ref.abs() + ref.abs().mean())).max().item()
        assert err < 0.02, (m, err)
    narrow = ops.prepare_weight(rnd((2 * 8192, 200), torch.bfloat16, 7, scale=0.05).cuda())       # K no multiple of 64
    calls.clear()
    ops.linear_swiglu(rnd((1024, 200), torch.bfloat16, 8).cuda(), narrow)
    assert not calls
    with pytest.raises(KernelError):
        real(rnd((1024, 200), torch.bfloat16, 8).cuda(), narrow, torch.empty((1024, 8192), dtype=torch.bfloat16, device="cuda"), ops._EPI_SWIGLU)


def test_large_bf16_product(ops):
    x = rnd((300, 256), torch.bfloat16, 3).cuda()
    w = rnd((520, 256), torch.bfloat16, 4).cuda()
    out = ops.linear(x, w, None, torch.bfloat16)
    assert close(out, x.double() @ w.double().t(), torch.bfloat16)


# ------------------------------------------------------------------------------- SiLU-mul
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [150, 152, 1024])              # src/flint/cuda/test.cc:208-211
def test_silu_mul(ops, dtype, width):
    gu = rnd((9, width), dtype, 15, 2.0).cuda()
    out = ops.silu_mul(gu)
    i = width // 2
    g, u = gu[:, :i].double(), gu[:, i:].double()
    ref = g / (1 + torch.exp(-g)) * u
    assert close(out, ref, dtype, f32=2e-6)
    swapped = u / (1 + torch.exp(-u)) * g                          # gating the wrong half must differ
    assert not close(out, swapped, dtype, f32=1e-2, bf16=1e-2)


def test_silu_mul_limits(ops):
    gu = torch.tensor([[0.0, 30.0, -30.0, 5.0, 3.0, 2.0, 7.0, 11.0]], device="cuda")
    out = ops.silu_mul(gu).cpu()
    assert out[0, 0] == 0.0                                        # gate 0 -> 0
    assert abs(out[0, 1] - 30.0 * 2.0) < 1e-4                      # large gate -> gate * up
    assert abs(out[0, 2]) < 1e-10


def test_silu_mul_limits_bfloat16_vectors(ops):
    # the vector kernel computes 1 / (1 + 2^(-g log2 e)) with the hardware's exp2 and reciprocal:
    # a gate far below zero overflows the power to infinity, and the product must be 0, not NaN
    gates = [0.0, 30.0, -30.0, 5.0, -100.0, -1000.0, 100.0, 1.0]
    ups = [3.0, 2.0, 7.0, 11.0, 5.0, 5.0, 0.5, -4.0]
    gu = torch.tensor([gates + ups], device="cuda", dtype=torch.bfloat16)
    out = ops.silu_mul(gu).float().cpu()[0]
    assert torch.isfinite(out).all()
    assert out[0] == 0.0 and out[2].abs() < 1e-9 and out[4] == 0.0 and out[5] == 0.0
    assert out[1] == 60.0 and out[6] == 50.0
    g, u = torch.tensor(gates, dtype=torch.float64), torch.tensor(ups, dtype=torch.float64)
    assert close(out, g / (1 + torch.exp(-g)) * u, torch.bfloat16)


# ------------------------------------------------------------------------------- rotation + cache write
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(4, 2, 16, 16), (6, 1, 32, 32), (6, 3, 48, 24), (5, 5, 80, 80), (32, 8, 64, 0)])
@pytest.mark.parametrize("bias", [False, True])
def test_rope_kv_write(ops, dtype, shape, bias):
    n_heads, n_kv, hd, rot = shape
    seqs = [(2, 0, 5), (0, 61, 9), (1, 130, 1)]                   # crosses page borders
    ctx = make_ctx(ops, dtype, seqs)
    kv = make_kv("cuda", dtype, 3, 4, n_kv, hd, seed=1)
    m = ctx.n_tokens
    width = (n_heads + 2 * n_kv) * hd
    qkv = rnd((m, width), dtype, 16).cuda()
    b = rnd((width,), torch.float32, 17).cuda() if bias else None
    half = rot // 2
    inv = 1.0 / (10000.0 ** (torch.arange(0, rot, 2, dtype=torch.float64) / max(rot, 1)))
    ang = torch.arange(300, dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = (torch.cos(ang).float().cuda(), torch.sin(ang).float().cuda()) if rot else (None, None)
    x = qkv.double().cpu() + (b.double().cpu() if bias else 0)
    ops.rope_kv_write(qkv, b, n_heads, n_kv, hd, cos, sin, rot, ctx, kv, True)
    pos = ctx.tok_pos.cpu().long()
    heads = x[:, :(n_heads + n_kv) * hd].reshape(m, n_heads + n_kv, hd).clone()
    if rot:
        c, s = torch.cos(ang)[pos][:, None, :], torch.sin(ang)[pos][:, None, :]
        x1, x2 = heads[..., :half].clone(), heads[..., half:rot].clone()
        heads[..., :half] = x1 * c - x2 * s
        heads[..., half:rot] = x2 * c + x1 * s
    tol = dict(f32=2e-6)
    assert close(qkv[:, :n_heads * hd], heads[:, :n_heads].reshape(m, -1), dtype, **tol)
    o = 0
    for slot, p0, n in seqs:
        k_got, v_got = read_kv(kv, slot, p0 + n)
        assert close(k_got[p0:], heads[o:o + n, n_heads:], dtype, **tol)
        v_ref = x[o:o + n, (n_heads + n_kv) * hd:].reshape(n, n_kv, hd)
        assert close(v_got[p0:], v_ref, dtype, **tol)
        assert torch.count_nonzero(k_got[:p0]) == 0               # nothing else is touched
        o += n


def pair_order(n_heads, n_kv, hd, rot):
    """Rows of a stacked q|k|v projection with the dims of a rotating pair side by side."""
    head = torch.arange(hd)
    head[0:rot:2] = torch.arange(rot // 2)
    head[1:rot:2] = torch.arange(rot // 2) + rot // 2
    qk = (torch.arange(n_heads + n_kv)[:, None] * hd + head[None, :]).reshape(-1)
    return torch.cat([qk, torch.arange((n_heads + n_kv) * hd, (n_heads + 2 * n_kv) * hd)])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(4, 2, 16, 16), (6, 3, 48, 24), (32, 8, 64, 64), (3, 1, 32, 0)])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("seqs", [[(2, 0, 5), (0, 61, 9), (1, 130, 1)], [(1, 63, 1), (0, 0, 1), (2, 200, 1)]])
def test_projection_with_rotation_and_cache_write(ops, dtype, shape, bias, seqs):
    """The q|k|v projection, rotation and cache write in one call (one kernel for few rows in
    bfloat16, from a matrix and from rows still to be normalised) against the plain formulas on the rows in their
    natural order; the two pairings hold the same numbers in different places."""
    n_heads, n_kv, hd, rot = shape
    k_in = 72
    ctx = make_ctx(ops, dtype, seqs)
    m = ctx.n_tokens
    n = (n_heads + 2 * n_kv) * hd
    x = rnd((m, k_in), torch.bfloat16, 40)
    w = rnd((n, k_in), torch.bfloat16, 41, 0.2)
    b = rnd((n,), torch.float32, 42) if bias else None
    order = pair_order(n_heads, n_kv, hd, rot) if rot else torch.arange(n)
    half = rot // 2
    inv = 1.0 / (10000.0 ** (torch.arange(0, rot, 2, dtype=torch.float64) / max(rot, 1)))
    ang = torch.arange(300, dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = (torch.cos(ang).float().cuda(), torch.sin(ang).float().cuda()) if rot else (None, None)
    # the plain result, natural order
    y = x.double() @ w.double().t() + (b.double() if bias else 0)
    pos = ctx.tok_pos.cpu().long()
    heads = y[:, :(n_heads + n_kv) * hd].reshape(m, n_heads + n_kv, hd).clone()
    if rot:
        c, s_ = torch.cos(ang)[pos][:, None, :], torch.sin(ang)[pos][:, None, :]
        x1, x2 = heads[..., :half].clone(), heads[..., half:rot].clone()
        heads[..., :half] = x1 * c - x2 * s_
        heads[..., half:rot] = x2 * c + x1 * s_
    v_ref = y[:, (n_heads + n_kv) * hd:].reshape(m, n_kv, hd)
    head_order = order[:hd]                                    # where each dim of a head went
    wd = w.cuda().to(dtype)[order.cuda()].contiguous()
    bd = b.cuda()[order.cuda()].contiguous() if bias else None
    tol = dict(f32=2e-5, bf16=2 * BF16_2ULP)
    for lazy in (False, True):
        kv = make_kv("cuda", dtype, 3, 4, n_kv, hd, seed=1)
        if lazy:                                               # the input as rows still to be normalised
            stream = (x.float() * 3.0).cuda()
            stream[0] *= 50.0
            wn = (1.0 + 0.3 * rnd((k_in,), torch.float32, 43)).cuda()
            xin = ops.normed(stream, wn, 1e-5)
            sd = stream.double().cpu()
            hn = sd * wn.double().cpu() / torch.sqrt((sd * sd).mean(-1, keepdim=True) + 1e-5)
            scale = None
        else:
            xin = x.cuda().to(dtype)
        if lazy:
            y2 = hn @ w.double().t() + (b.double() if bias else 0)
            heads2 = y2[:, :(n_heads + n_kv) * hd].reshape(m, n_heads + n_kv, hd).clone()
            if rot:
                x1, x2 = heads2[..., :half].clone(), heads2[..., half:rot].clone()
                heads2[..., :half] = x1 * c - x2 * s_
                heads2[..., half:rot] = x2 * c + x1 * s_
            want_heads, want_v = heads2, y2[:, (n_heads + n_kv) * hd:].reshape(m, n_kv, hd)
        else:
            want_heads, want_v = heads, v_ref
        out = ops.qkv_rope(xin, wd, bd, n_heads, n_kv, hd, cos, sin, rot, ctx, kv, True, bool(rot), dtype)
        q = out[:, :n_heads * hd].reshape(m, n_heads, hd)
        assert close(q, want_heads[:, :n_heads][..., head_order], dtype, **tol)
        o = 0
        for slot, p0, n_new in seqs:
            k_got, v_got = read_kv(kv, slot, p0 + n_new)
            assert close(k_got[p0:], want_heads[o:o + n_new, n_heads:][..., head_order], dtype, **tol)
            assert close(v_got[p0:], want_v[o:o + n_new], dtype, **tol)
            assert torch.count_nonzero(k_got[:p0]) == 0 and torch.count_nonzero(v_got[:p0]) == 0
            o += n_new
    # queries alone, for a layer that reads another layer's keys
    kv = make_kv("cuda", dtype, 3, 4, n_kv, hd, seed=1)
    q_only = ops.qkv_rope(x.cuda().to(dtype), wd[:n_heads * hd].contiguous(), bd, n_heads, n_kv, hd, cos, sin,
                          rot, ctx, kv, False, bool(rot), dtype)
    assert close(q_only[:, :n_heads * hd].reshape(m, n_heads, hd), heads[:, :n_heads][..., head_order], dtype, **tol)
    assert torch.count_nonzero(kv.plane("k")) == 0


@pytest.mark.parametrize("shape", [(4, 2, 16, 16), (6, 3, 48, 24), (5, 1, 64, 64), (8, 2, 128, 128), (2, 2, 256, 64),
                                   (3, 1, 32, 0)])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("seqs", [
    [(2, 0, 70), (0, 61, 9), (1, 130, 50), (3, 5, 31)],            # 160 rows: two tiles and a half
    [(2, 0, 200), (0, 61, 90), (1, 130, 60)],                      # 350 rows: a v head is one block's again
    [(i, (37 * i) % 250, 1) for i in range(70)],                   # a decode step: every row in a page of its own
], ids=["160rows", "350rows", "70decode"])
def test_rope_kv_write_on_many_rows(ops, shape, bias, seqs):
    """Steps of 64 rows and more in bfloat16 with neighbouring pairs take a kernel of their own (tiles
    of 64 rows, v transposed through LDS, a v head dealt to several blocks where the rows are few):
    several sequences that cross page borders, a last tile that is not full, partial rotation, rows of
    as many sequences; and nothing beside the new positions is written."""
    n_heads, n_kv, hd, rot = shape
    dtype = torch.bfloat16
    n_slots = max(slot for slot, _, _ in seqs) + 1
    ctx = make_ctx(ops, dtype, seqs)
    m = ctx.n_tokens
    width = (n_heads + 2 * n_kv) * hd
    nat = rnd((m, width), dtype, 50)                                # rows in their natural order
    b_nat = rnd((width,), torch.float32, 51) if bias else None
    order = pair_order(n_heads, n_kv, hd, rot) if rot else torch.arange(width)
    head_order = order[:hd]
    half = rot // 2
    inv = 1.0 / (10000.0 ** (torch.arange(0, rot, 2, dtype=torch.float64) / max(rot, 1)))
    ang = torch.arange(300, dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = (torch.cos(ang).float().cuda(), torch.sin(ang).float().cuda()) if rot else (None, None)
    x = nat.double() + (b_nat.double() if bias else 0)
    pos = ctx.tok_pos.cpu().long()
    heads = x[:, :(n_heads + n_kv) * hd].reshape(m, n_heads + n_kv, hd).clone()
    if rot:
        c, s_ = torch.cos(ang)[pos][:, None, :], torch.sin(ang)[pos][:, None, :]
        x1, x2 = heads[..., :half].clone(), heads[..., half:rot].clone()
        heads[..., :half] = x1 * c - x2 * s_
        heads[..., half:rot] = x2 * c + x1 * s_
    v_ref = x[:, (n_heads + n_kv) * hd:].reshape(m, n_kv, hd)
    for write in (True, False):
        kv = make_kv("cuda", dtype, n_slots, 4, n_kv, hd, seed=1)
        cols = width if write else n_heads * hd                     # queries alone when nothing is written
        qkv = nat[:, order][:, :cols].contiguous().cuda()
        bd = b_nat[order][:cols].contiguous().cuda() if bias else None
        ops.rope_kv_write(qkv, bd, n_heads, n_kv, hd, cos, sin, rot, ctx, kv, write, adjacent=bool(rot))
        q = qkv[:, :n_heads * hd].reshape(m, n_heads, hd)
        assert close(q, heads[:, :n_heads][..., head_order], dtype)
        if not write:
            assert torch.count_nonzero(kv.plane("k")) == 0 and torch.count_nonzero(kv.plane("v")) == 0
            continue
        o = 0
        for slot, p0, n_new in seqs:
            k_got, v_got = read_kv(kv, slot, p0 + n_new)
            assert close(k_got[p0:], heads[o:o + n_new, n_heads:][..., head_order], dtype)
            assert close(v_got[p0:], v_ref[o:o + n_new], dtype)
            assert torch.count_nonzero(k_got[:p0]) == 0 and torch.count_nonzero(v_got[:p0]) == 0
            o += n_new
        written = sum(n for _, _, n in seqs) * n_kv * hd
        assert torch.count_nonzero(kv.plane("k")) <= written and torch.count_nonzero(kv.plane("v")) <= written


def test_rope_pairing_and_sign(ops):
    # a unit vector in dimension 0 at position p becomes cos at 0 and +sin at hd/2:
    # o[j] = x[j] c - x[j+hd/2] s, o[j+hd/2] = x[j+hd/2] c + x[j] s   (src/libllm/llama.cc:151-176)
    hd = 16
    ctx = make_ctx(ops, torch.float32, [(0, 3, 1)])
    kv = make_kv("cuda", torch.float32, 1, 1, 1, hd)
    qkv = torch.zeros((1, 3 * hd), device="cuda")
    qkv[0, 0] = 1.0
    theta = 0.7
    cos = torch.full((8, hd // 2), math.cos(theta), device="cuda")
    sin = torch.full((8, hd // 2), math.sin(theta), device="cuda")
    ops.rope_kv_write(qkv, None, 1, 1, hd, cos, sin, hd, ctx, kv, True)
    q = qkv[0, :hd].cpu()
    assert abs(q[0] - math.cos(theta)) < 1e-6 and abs(q[hd // 2] - math.sin(theta)) < 1e-6
    assert torch.count_nonzero(q) == 2


# ------------------------------------------------------------------------------- attention
def run_attention(ops, dtype, n_heads, n_kv, hd, seqs, window=0, seed=0, boost=None, fast=True, tiles=0,
                  checked=None, unequal=False):
    """seqs: (slot, past, new).  Returns (out, oracle) over all new tokens, or, with ``checked``,
    over that many rows of every sequence (its first and last, those next to every border of a
    block of 128 rows among them, the others drawn)."""
    ctx = make_ctx(ops, dtype, seqs)
    ctx.unequal = unequal                              # decode attention deals its pages out by length
    pages = max((p + n + PAGE - 1) // PAGE for _, p, n in seqs)
    kv = make_kv("cuda", dtype, max(s for s, _, _ in seqs) + 1, pages, n_kv, hd, seed=seed)
    scale = hd ** -0.5
    q = rnd((ctx.n_tokens, n_heads * hd + 24), dtype, seed + 1)   # wider rows: a stride is honoured
    ref, rows, o = [], [], 0
    for slot, past, new in seqs:
        keys = rnd((past + new, n_kv, hd), dtype, seed + 10 + slot)
        vals = rnd((past + new, n_kv, hd), dtype, seed + 20 + slot)
        if boost is not None:                                       # one far key stands out
            key_pos, gain = boost
            if key_pos < past + new:                                # (a sequence too short for it has none)
                keys[key_pos] = keys[key_pos] * gain
        fill_kv(kv, slot, keys, vals)
        which = range(new)
        if checked is not None and new > checked:
            g = np.random.default_rng(seed + slot)
            edge = [t for b in (g.integers(1, max(2, new // 128), size=4) * 128).tolist() for t in (b - 1, b)]
            which = sorted({0, new - 1, *[t for t in edge if 0 <= t < new],
                            *g.integers(0, new, size=checked).tolist()})[:checked + 10]
        keys, vals = keys.double(), vals.double()
        for t in which:
            qt = q[o + t, :n_heads * hd].double().reshape(n_heads, hd)
            ref.append(attention_oracle(qt, keys, vals, past + t, scale, window).reshape(-1))
            rows.append(o + t)
        o += new
    ops.fast_attention, ops.prompt_tiles = fast, tiles
    try:
        out = ops.attention(q.cuda(), n_heads, n_kv, hd, ctx, kv, scale, window)
    finally:
        ops.fast_attention, ops.prompt_tiles = True, 0
    return out[torch.tensor(rows, device=out.device)].double().cpu(), torch.stack(ref)


# (heads, kv heads, queries, keys, head size): the cases of src/flint/cuda/test.cc:349-362
REFERENCE_CASES = [(8, 8, 8, 8, 128), (8, 8, 128, 128, 128), (8, 2, 6, 10, 128), (8, 2, 1, 10, 128),
                   (8, 2, 1, 2048, 128), (8, 2, 4, 1024, 128), (8, 8, 16, 16, 16), (8, 2, 6, 10, 16)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", REFERENCE_CASES)
def test_attention_reference_cases(ops, dtype, case):
    n_heads, n_kv, lq, lk, hd = case
    out, ref = run_attention(ops, dtype, n_heads, n_kv, hd, [(0, lk - lq, lq)])
    assert max_err(out, ref) < (1e-5 if dtype == torch.float32 else BF16_2ULP)


@pytest.mark.parametrize("fast", [True, False])
@pytest.mark.parametrize("hd", list(range(16, 257, 16)))
def test_attention_head_sizes_bf16(ops, hd, fast):
    # unequal batch: a fresh prompt, a continued one crossing pages, a single token with a long past
    seqs = [(1, 0, 70), (0, 100, 37), (2, 300, 1)]
    out, ref = run_attention(ops, torch.bfloat16, 6, 3, hd, seqs, seed=hd, fast=fast)
    assert max_err(out, ref) < BF16_2ULP


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("groups", [(5, 5), (6, 1), (20, 1), (12, 4), (3, 3)])
def test_attention_groups_decode_and_prefill(ops, dtype, groups):
    n_heads, n_kv = groups
    for seqs in ([(0, 129, 1), (1, 0, 1), (2, 64, 1), (3, 63, 1)],          # decode: one token each
                 [(0, 129, 3), (1, 0, 65)]):
        out, ref = run_attention(ops, dtype, n_heads, n_kv, 64, seqs, seed=3)
        assert max_err(out, ref) < (1e-5 if dtype == torch.float32 else BF16_2ULP)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 5, 64, 65, 200])
def test_attention_window(ops, dtype, window):
    for seqs in ([(0, 0, 150)], [(0, 333, 1), (1, 64, 1)], [(0, 190, 20)]):
        out, ref = run_attention(ops, dtype, 4, 2, 32, seqs, window=window, seed=window)
        assert max_err(out, ref) < (1e-5 if dtype == torch.float32 else BF16_2ULP)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("far", [0, 3, 63, 64, 700])
def test_attention_far_key_stands_out(ops, dtype, far):
    """With random scores a lost key among hundreds changes little; here one key's score is made
    to dominate, so that dropping or misplacing it cannot pass."""
    for seqs in ([(0, 900, 1)], [(0, 0, 901)]):
        out, ref = run_attention(ops, dtype, 4, 2, 64, seqs, seed=9, boost=(far, 12.0))
        assert max_err(out, ref) < (1e-5 if dtype == torch.float32 else BF16_2ULP)


@pytest.mark.parametrize("tiles", [1, 2])
@pytest.mark.parametrize("hd,window", [(16, 0), (64, 0), (64, 70), (80, 5), (128, 0), (128, 130), (144, 0), (176, 90),
                                       (208, 0), (240, 0), (256, 64)])
def test_prompt_attention_tiles_of_rows(ops, hd, window, tiles):
    """A wave of the prompt kernel takes one or two tiles of 16 rows (blocks of 64 or 128 rows),
    by the number of blocks; here both are forced on small cases: prompts that end inside the first
    and inside the second half of a block, a continued one that crosses pages, a single token, and
    windows shorter and longer than a block."""
    seqs = [(1, 0, 70), (0, 100, 137), (2, 300, 1), (3, 0, 200), (4, 40, 128)]
    out, ref = run_attention(ops, torch.bfloat16, 6, 3, hd, seqs, window=window, seed=hd + window, tiles=tiles)
    assert max_err(out, ref) < BF16_2ULP
    out, ref = run_attention(ops, torch.bfloat16, 4, 2, hd, [(0, 0, 901)], window=window, seed=9,
                             boost=(63 if window else 700, 12.0), tiles=tiles)
    assert max_err(out, ref) < BF16_2ULP


def test_prompt_attention_takes_two_tiles_for_long_prompts(ops):
    """Left to itself the launcher takes two tiles a wave where the longest sequence brings 3,584
    rows or more (head size 64); a row's bits do not depend on it."""
    n_heads, n_kv, hd, rows = 32, 8, 64, 3600
    seqs = [(0, 0, rows), (1, 64, 500)]
    assert rows >= ops.PROMPT_TILE_ROWS[0]
    ctx = make_ctx(ops, torch.bfloat16, seqs)
    kv = make_kv("cuda", torch.bfloat16, 2, (rows + 64) // PAGE + 1, n_kv, hd, seed=2)
    kv.plane("k").normal_(); kv.plane("v").normal_()
    q = rnd((ctx.n_tokens, n_heads * hd), torch.bfloat16, 5).cuda()
    outs = []
    for tiles in (0, 1, 2):
        ops.prompt_tiles = tiles
        try:
            outs.append(ops.attention(q, n_heads, n_kv, hd, ctx, kv, hd ** -0.5, 0))
        finally:
            ops.prompt_tiles = 0
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    assert outs[0].float().abs().max() < 10 and torch.isfinite(outs[0].float()).all()


@pytest.mark.parametrize("ctx_len,far", [(2100, 5), (9000, 4321), (9000, 8999)])
def test_attention_decode_over_many_pages(ops, ctx_len, far):
    """A decoded token over thousands of keys: the pages are dealt out to many blocks whose
    partial results a second kernel merges (through each of its variants); one far key dominates."""
    out, ref = run_attention(ops, torch.bfloat16, 8, 2, 64, [(0, ctx_len, 1)], seed=3, boost=(far, 12.0))
    assert max_err(out, ref) < BF16_2ULP
    out, ref = run_attention(ops, torch.bfloat16, 4, 1, 128, [(1, ctx_len // 2, 1), (0, ctx_len, 1)], seed=4)
    assert max_err(out, ref) < BF16_2ULP


@pytest.mark.parametrize("hd", [64, 128])
@pytest.mark.parametrize("ctx_len,far", [(32768, 17), (131072, 70001), (131072, 131071)])
def test_attention_decode_over_tens_of_thousands_of_keys(ops, hd, ctx_len, far):
    """Contexts at which the measurements run and whose grids differ from the shorter ones': a
    wave walks several pages in a row, and at 131,072 keys the merge is its loop form.  One
    sequence with one far key that dominates, then eight of unequal lengths in one step."""
    out, ref = run_attention(ops, torch.bfloat16, 8, 2, hd, [(0, ctx_len - 1, 1)], seed=hd, boost=(far, 12.0))
    assert max_err(out, ref) < BF16_2ULP
    lens = [ctx_len - 1, 5, ctx_len // 2 + 33, 4097, ctx_len - 64, 63, ctx_len // 3, 20000]
    out, ref = run_attention(ops, torch.bfloat16, 4, 2, hd, [(i, n, 1) for i, n in enumerate(lens)], seed=hd + 5)
    assert max_err(out, ref) < BF16_2ULP


@pytest.mark.parametrize("tiles", [1, 2])
@pytest.mark.parametrize("hd,rows", [(64, 8192), (128, 8192), (64, 16384), (128, 16384)])
def test_prompt_attention_over_thousands_of_rows(ops, hd, rows, tiles):
    """Prompts as long as the measured ones, in both forms of the kernel (one and two tiles of
    rows a wave): some hundred rows of a fresh prompt against the oracle, one far key dominating;
    then a prompt that continues a sequence, beside a short one."""
    out, ref = run_attention(ops, torch.bfloat16, 4, 2, hd, [(0, 0, rows)], seed=rows + hd, boost=(rows // 3, 12.0),
                             tiles=tiles, checked=120)
    assert max_err(out, ref) < BF16_2ULP
    out, ref = run_attention(ops, torch.bfloat16, 6, 2, hd, [(1, 0, 70), (0, 1000, rows - 1500)], seed=rows + hd + 1,
                             tiles=tiles, checked=60)
    assert max_err(out, ref) < BF16_2ULP


def test_a_build_whose_product_for_33_to_128_rows_spills_does_not_use_it(monkeypatch):
    """The build's record decides (see test_build.py): with a spill on record the host sends
    steps of 33 to 128 rows to the product for few rows and to the library's."""
    from libllm_amd.hip import HipOps, build
    assert HipOps().mid_gemm
    monkeypatch.setattr(build, "trusted", lambda source, path=None: False)
    other = HipOps()
    assert not other.mid_gemm
    x, w = rnd((100, 256), torch.bfloat16, 1).cuda(), rnd((3200, 256), torch.bfloat16, 2).cuda()
    assert not other._mid_ok(x, other.prepare_weight(w), 100, 256)


BY_LENGTH = {
    "one long among short": [(0, 9000, 1), (1, 3, 1), (2, 70, 1), (3, 0, 1), (4, 64, 1)],
    "two long": [(0, 5000, 1), (1, 63, 1), (2, 4999, 1)],
    "all equal": [(i, 700, 1) for i in range(6)],
    "all short": [(i, i, 1) for i in range(9)],
    "seventy sequences": [(i, (37 * i) % 300 if i != 50 else 6000, 1) for i in range(70)],
    "two hundred sequences": [(i, (53 * i) % 200 if i % 67 else 3000 + i, 1) for i in range(200)],
}


@pytest.mark.parametrize("case", list(BY_LENGTH))
@pytest.mark.parametrize("shape", [(8, 2, 64), (4, 4, 128), (20, 1, 32), (2, 1, 256), (6, 3, 176)])
def test_attention_decode_by_length(ops, case, shape):
    """Decode attention with its pages dealt out by the sequences' lengths (a flat grid, every
    block finding its share from the lengths in device memory): one long sequence among short
    ones, equal ones, more sequences than a wave has lanes; groups of 4, 1 and 20 heads, heads of
    32 to 256 dims; against the per-query oracle, and the same bits as the uniform grid gives
    where a pair is one chunk in both."""
    n_heads, n_kv, hd = shape
    seqs = BY_LENGTH[case]
    if hd >= 176:
        seqs = seqs[:40]                                  # (the oracle is slow)
    out, ref = run_attention(ops, torch.bfloat16, n_heads, n_kv, hd, seqs, seed=len(seqs) + hd, unequal=True)
    assert max_err(out, ref) < BF16_2ULP
    far = max(range(len(seqs)), key=lambda i: seqs[i][1])
    out, ref = run_attention(ops, torch.bfloat16, n_heads, n_kv, hd, seqs, seed=hd, unequal=True,
                             boost=(seqs[far][1] // 2, 12.0))
    assert max_err(out, ref) < BF16_2ULP


@pytest.mark.parametrize("window", [0, 100, 4096])
def test_attention_decode_by_length_with_a_window(ops, window):
    seqs = [(0, 9000, 1), (1, 3, 1), (2, 70, 1), (3, 5000, 1), (4, 64, 1)]
    out, ref = run_attention(ops, torch.bfloat16, 8, 2, 64, seqs, window=window, seed=5, unequal=True)
    assert max_err(out, ref) < BF16_2ULP


@pytest.mark.parametrize("hd", [144, 160, 176, 192, 208, 224, 240, 256])
@pytest.mark.parametrize("ctx_len,far", [(600, 3), (2100, 1999), (9000, 77)])
def test_attention_decode_of_wide_heads_over_many_pages(ops, hd, ctx_len, far):
    """Heads wider than 128: the decode kernel without its overlap of pages (four waves a block
    up to head size 192, two beyond), and each form of the
    merge (up to 8 partials, up to 32, and the loop, whose block must stay within 1,024 threads:
    four groups of 192 or 256 threads, not eight).  One far key dominates."""
    out, ref = run_attention(ops, torch.bfloat16, 4, 2, hd, [(0, ctx_len, 1)], seed=hd, boost=(far, 12.0))
    assert max_err(out, ref) < BF16_2ULP
    out, ref = run_attention(ops, torch.bfloat16, 2, 1, hd, [(1, ctx_len - 70, 1), (0, ctx_len, 1)], seed=hd + 1)
    assert max_err(out, ref) < BF16_2ULP


@pytest.mark.parametrize("hd", [64, 128])
@pytest.mark.parametrize("blocks", [1, 3, 4096])
def test_attention_decode_pages_of_a_wave(ops, monkeypatch, hd, blocks):
    """With few blocks a wave walks many pages, asking for the next while it works on one (grids
    of up to two blocks a compute unit); with many sequences and kv heads the grid is larger and
    the kernel's other form runs.  One far key dominates; a window cuts the walk short."""
    monkeypatch.setattr(ops, "DECODE_BLOCKS", blocks)
    monkeypatch.setattr(ops, "DECODE_BLOCKS_AHEAD", min(blocks, 512))
    for window in (0, 700):
        out, ref = run_attention(ops, torch.bfloat16, 8, 2, hd, [(0, 2100, 1), (1, 2030, 1)], window=window,
                                 seed=blocks, boost=(2000, 10.0))
        assert max_err(out, ref) < BF16_2ULP


def test_attention_decode_on_a_large_grid(ops):
    """More (sequence, kv head) pairs than two blocks a compute unit: the form of the kernel that
    loads a page, then computes.  Against the oracle."""
    n_kv, seqs = 16, [(i, 70 + 9 * i, 1) for i in range(40)]
    assert len(seqs) * n_kv > 512
    out, ref = run_attention(ops, torch.bfloat16, 16, n_kv, 64, seqs, seed=8)
    assert max_err(out, ref) < BF16_2ULP


def test_attention_single_token_is_value(ops):
    # one query, no past: the output is the value itself
    out, ref = run_attention(ops, torch.float32, 4, 4, 32, [(0, 0, 1)])
    assert max_err(out, ref) < 1e-6


# ------------------------------------------------------------------------------- sampling
def test_argmax_reference_vectors(ops):
    # src/flint/cuda/test.cc:376-392
    p = torch.tensor([[0.4, 0.3, 0.2, 0.1], [0.1, 0.2, 0.6, 0.1], [0.05, 0.05, 0.1, 0.8]]).cuda()
    assert ops.argmax(p).tolist() == [0, 2, 3]
    # src/flint/cuda/test.cc:405-415: the maximum lies beyond the first block of the row
    v = torch.zeros((2, 2050))
    v[0, 2049], v[1, 1100] = 0.4, 0.7
    assert ops.argmax(v.cuda()).tolist() == [2049, 1100]
    t = torch.zeros((1, 5000))
    t[0, 17] = t[0, 4000] = t[0, 999] = 3.0                                 # ties: lowest index
    assert ops.argmax(t.cuda()).tolist() == [17]


def test_sampling_matches_plain(ops):
    from plain import sampling
    g = torch.Generator().manual_seed(21)
    for vocab, top_k, top_p, temp in [(1000, 50, 0.8, 0.8), (517, 0, 1.0, 1.3), (128256, 50, 0.9, 1.0),
                                      (300, 300, 0.5, 0.7), (2050, 1024, 0.95, 2.0), (64, 7, 1.0, 0.5)]:
        logits = (torch.randn((24, vocab), generator=g) * 3.0)
        streams = list(range(100, 124))
        counters = list(range(24))
        k = 0 if top_k >= vocab else top_k
        got = ops.sample(logits.cuda(), temp, k, top_p, 77, streams, counters).tolist()
        bad = 0
        for r in range(24):
            u = sampling.uniform(77, streams[r], counters[r])
            want = sampling.sample(logits[r].double().numpy(), temp, k, top_p, u)
            if got[r] != want:
                # only a draw within rounding of a boundary of the running sum may differ
                assert sampling.margin(logits[r].double().numpy(), temp, k, top_p, u) < 1e-5, (vocab, r)
                bad += 1
        assert bad <= 2


def test_sampling_with_many_equal_logits(ops):
    """Logits of few distinct values: the top-k cut falls inside a run of equal ones (the lowest
    indices are kept), or takes a whole run (where the selection stops early)."""
    from plain import sampling
    g = torch.Generator().manual_seed(5)
    for vocab, top_k, top_p, temp, step in [(3000, 50, 0.9, 1.0, 1.0), (128256, 50, 0.8, 1.0, 0.5),
                                            (9000, 200, 1.0, 0.7, 2.0), (5000, 64, 0.95, 1.5, 4.0)]:
        logits = torch.round(torch.randn((16, vocab), generator=g) * 3.0 / step) * step
        streams, counters = list(range(16)), list(range(50, 66))
        got = ops.sample(logits.cuda(), temp, top_k, top_p, 9, streams, counters).tolist()
        bad = 0
        for r in range(16):
            u = sampling.uniform(9, streams[r], counters[r])
            want = sampling.sample(logits[r].double().numpy(), temp, top_k, top_p, u)
            if got[r] != want:
                assert sampling.margin(logits[r].double().numpy(), temp, top_k, top_p, u) < 1e-5, (vocab, r)
                bad += 1
        assert bad <= 2, (vocab, bad)


def test_sampling_takes_both_zeros_for_one_value(ops):
    """Logits of -0.0 and +0.0 are equal: among equal logits the lower index comes first, whatever
    the sign of a zero (a kernel that orders by the bits of the float puts every +0 before every -0)."""
    from plain import sampling
    g = torch.Generator().manual_seed(11)
    for vocab, top_k, top_p, temp in [(300, 50, 0.95, 1.6), (188, 0, 0.8, 0.7), (2007, 1000, 0.8, 0.7), (260, 200, 0.95, 0.3),
                                      (5000, 0, 1.0, 1.0)]:
        logits = torch.round(torch.randn((32, vocab), generator=g) * 0.5)       # -1, -0.0, 0.0, 1 for the most part
        assert (logits == 0).sum() > vocab and torch.signbit(logits[logits == 0]).any() and not torch.signbit(logits[logits == 0]).all()
        streams, counters = list(range(32)), list(range(200, 232))
        got = ops.sample(logits.cuda(), temp, top_k, top_p, 21, streams, counters).tolist()
        for r in range(32):
            u = sampling.uniform(21, streams[r], counters[r])
            want = sampling.sample(logits[r].double().numpy(), temp, top_k, top_p, u)
            if got[r] != want:
                assert sampling.margin(logits[r].double().numpy(), temp, top_k, top_p, u) < 1e-5, (vocab, r, got[r], want)


@pytest.mark.parametrize("vocab", [5003, 128256])
def test_nucleus_without_a_limit_on_the_candidates(ops, vocab):
    """top_k 0 with top_p below 1 (the reference's sampler takes any top_k up to the vocabulary,
    src/libllm/generator.cc:66-90): the nucleus is the shortest prefix, in falling probability,
    that reaches top_p, however long.  Rows whose nucleus lies within the most probable 1,024
    tokens, rows as flat as to need most of the vocabulary (the walk over the whole vocabulary),
    a row of few distinct values (equal logits are ranked by index), and flat rows in which a
    third of the tokens are ruled out by a logit of minus infinity."""
    from plain import sampling
    g = torch.Generator().manual_seed(vocab)
    peaked = torch.randn((8, vocab), generator=g) * 4.0
    flat = torch.randn((8, vocab), generator=g) * 0.3
    stepped = torch.randint(0, 3, (8, vocab), generator=g).float() * 1.5
    holes = torch.randn((4, vocab), generator=g) * 0.3             # flat, with a third of the tokens ruled out
    holes[:, ::3] = -math.inf
    logits = torch.cat([peaked, flat, stepped, holes])
    rows = logits.shape[0]
    streams, counters = list(range(50, 50 + rows)), list(range(rows))
    # a row in which nothing has any probability decides nothing, and still names a token
    nothing = torch.full((2, vocab), -math.inf)
    got = ops.sample(nothing.cuda(), 1.0, 0, 0.9, 99, [1, 2], [0, 0]).tolist()
    assert all(0 <= t < vocab for t in got)
    for top_p, temp in ((0.9, 1.0), (0.5, 0.7), (0.999, 1.5)):
        got = ops.sample(logits.cuda(), temp, 0, top_p, 99, streams, counters).tolist()
        bad, long_ones = 0, 0
        for r in range(rows):
            row = logits[r].double().numpy()
            u = sampling.uniform(99, streams[r], counters[r])
            labels, _ = sampling.candidates(row, temp, 0, top_p)
            long_ones += len(labels) > 1024
            want = sampling.sample(row, temp, 0, top_p, u)
            if got[r] != want:
                # only a draw within rounding of a boundary of the running sum may differ (with equal
                # logits a boundary moves the pick to a neighbour of equal probability)
                assert sampling.margin(row, temp, 0, top_p, u) < 1e-5 and got[r] in labels, (vocab, top_p, r)
                bad += 1
        assert bad <= 2 and long_ones >= 8                      # the long walk was taken


def test_sampling_seed_and_top1(ops):
    g = torch.Generator().manual_seed(5)
    logits = torch.randn((6, 999), generator=g).cuda()
    a = ops.sample(logits, 1.0, 40, 0.9, 1234, [0] * 6, list(range(6))).tolist()
    b = ops.sample(logits, 1.0, 40, 0.9, 1234, [0] * 6, list(range(6))).tolist()
    assert a == b                                                           # src/flint/cuda/test.cc:394-403
    c = ops.sample(logits, 1.0, 40, 0.9, 1235, [0] * 6, list(range(6))).tolist()
    assert a != c
    top1 = ops.sample(logits, 1.0, 1, 1.0, 1, [0] * 6, list(range(6))).tolist()
    assert top1 == ops.argmax(logits).tolist()                              # top_k 1 is arg-max


def test_sampling_distribution(ops):
    # many draws of one row follow its probabilities
    logits = torch.tensor([[0.0, 1.0, 2.0, 3.0, -50.0]]).repeat(4000, 1).cuda()
    got = ops.sample(logits, 1.0, 0, 1.0, 3, [0] * 4000, list(range(4000))).cpu().numpy()
    freq = np.bincount(got, minlength=5) / 4000.0
    p = torch.softmax(logits[0].double().cpu(), 0).numpy()
    assert np.abs(freq - p).max() < 0.03
