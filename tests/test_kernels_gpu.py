"""Each kernel alone against a plain float32 PyTorch reference of the same op, at sizes other
than the engine's test models: widths and vocabularies that are no power of two, head sizes
in steps of 16, odd head counts and groups, page sizes 8 to 64."""
import contextlib
import math

import numpy as np
import pytest
import torch

import plain_llama as plain
from rust_llm_inference_server_amd.stepplan import StepLengths

pytestmark = pytest.mark.gpu

DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype, f32=1e-4, bf16=2e-2):
    return dict(atol=f32, rtol=f32) if dtype == torch.float32 else dict(atol=bf16, rtol=bf16)


def rnd(*shape, dtype=torch.float32, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


@pytest.fixture(params=["matrix", "vector"])
def decode_kind(request):
    """Both decode attention kernels: on the matrix cores (bfloat16) and on the vector units."""
    from rust_llm_inference_server_amd import ops
    old = ops.DECODE_ATTENTION
    ops.DECODE_ATTENTION = request.param
    yield request.param
    ops.DECODE_ATTENTION = old


@pytest.fixture(scope="module")
def ops():
    from rust_llm_inference_server_amd import ops
    from rust_llm_inference_server_amd.ops import lib
    lib.load()
    assert lib.loaded_path().endswith("librlis_kernels.so")
    return ops


# ----------------------------------------------------------------------- rows
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("V,H,T", [(331, 100, 7), (1000, 2048, 33), (50, 3, 1)])
def test_embed(ops, dtype, V, H, T):
    table = rnd(V, H, dtype=dtype)
    ids = torch.randint(0, V, (T,), dtype=torch.int32, device=DEV)
    out = ops.embed(ids, table)
    assert out.dtype == torch.float32
    torch.testing.assert_close(out, table[ids.long()].float(), atol=0, rtol=0)


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("w_dtype", DTYPES)
@pytest.mark.parametrize("T,H,eps", [(5, 100, 1e-5), (3, 2048, 1e-6), (2, 8192, 1e-5), (1, 7, 0.1),
                                     (4, 3072, 1e-5), (3, 4104, 1e-6), (2, 1000, 1e-5), (2, 8200, 1e-5)])
def test_add_rmsnorm(ops, out_dtype, w_dtype, T, H, eps):
    resid = rnd(T, H, seed=1) * 3
    delta = rnd(T, H, dtype=out_dtype, seed=2)
    w = (1 + rnd(H, seed=3) * 0.1).to(w_dtype)
    want_resid = resid + delta.float()
    want = plain.rms_norm(want_resid.cpu(), w.float().cpu(), eps)
    r = resid.clone()
    out = ops.add_rmsnorm(r, delta, w, eps, out_dtype)
    torch.testing.assert_close(r, want_resid, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(out.float().cpu(), want, **tol(out_dtype, 2e-5))
    # no delta: plain norm, residual untouched
    r2 = resid.clone()
    out2 = ops.add_rmsnorm(r2, None, w, eps, out_dtype)
    torch.testing.assert_close(r2, resid, atol=0, rtol=0)
    torch.testing.assert_close(out2.float().cpu(), plain.rms_norm(resid.cpu(), w.float().cpu(), eps),
                               **tol(out_dtype, 2e-5))
    # selected rows with a pending delta: residual untouched, rows in the asked order
    rows = torch.tensor([T - 1, 0], dtype=torch.int32, device=DEV)
    r3 = resid.clone()
    out3 = ops.add_rmsnorm(r3, delta, w, eps, out_dtype, rows=rows)
    torch.testing.assert_close(r3, resid, atol=0, rtol=0)
    torch.testing.assert_close(out3.float().cpu(), want[[T - 1, 0]], **tol(out_dtype, 2e-5))


@pytest.mark.parametrize("out_dtype,w_dtype", [(torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32),
                                               (torch.float32, torch.float32)])
@pytest.mark.parametrize("T,H,parts", [(64, 2048, 16), (3, 100, 2), (17, 4096, 7), (5, 8192, 28), (2, 8196, 3),
                                       (9, 130, 5)])
def test_add_rmsnorm_of_a_stack_of_partial_sums(ops, out_dtype, w_dtype, T, H, parts):
    """The delta as a stack of float32 partial sums: they are added in order, their sum is
    rounded to bfloat16 when asked, then it joins the residual; with all rows and with a
    selection of rows; widths that take the vectorised kernel and widths that do not."""
    resid = rnd(T, H, seed=1) * 3
    stack = rnd(parts, T, H, seed=2)
    w = (1 + rnd(H, seed=3) * 0.1).to(w_dtype)
    for rounding in (False, True):
        total = stack[0].clone()
        for s in range(1, parts):
            total += stack[s]
        if rounding:
            total = total.to(torch.bfloat16).float()
        want_resid = resid + total
        want = plain.rms_norm(want_resid.cpu(), w.float().cpu(), 1e-5)
        r = resid.clone()
        out = ops.add_rmsnorm(r, stack, w, 1e-5, out_dtype, round_parts=rounding)
        assert torch.equal(r, want_resid)
        torch.testing.assert_close(out.float().cpu(), want, **tol(out_dtype, 2e-5))
        rows = torch.tensor([T - 1, 0], dtype=torch.int32, device=DEV)
        r3 = resid.clone()
        out3 = ops.add_rmsnorm(r3, stack, w, 1e-5, out_dtype, rows=rows, round_parts=rounding)
        assert torch.equal(r3, resid)
        torch.testing.assert_close(out3.float().cpu(), want[[T - 1, 0]], **tol(out_dtype, 2e-5))


def test_rmsnorm_unit_mean_square(ops):
    # with w = 1 and eps = 0 every row has unit mean square; scaling the input changes nothing
    x = rnd(4, 300, seed=5) * 7
    w = torch.ones(300, device=DEV)
    y = ops.add_rmsnorm(x.clone(), None, w, 0.0, torch.float32)
    torch.testing.assert_close((y * y).mean(-1), torch.ones(4, device=DEV), atol=1e-5, rtol=1e-5)
    y2 = ops.add_rmsnorm((x * 5).clone(), None, w, 0.0, torch.float32)
    torch.testing.assert_close(y, y2, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_add_residual(ops, dtype):
    r = rnd(9, 77, seed=1)
    d = rnd(9, 77, dtype=dtype, seed=2)
    want = r + d.float()
    ops.add_residual(r, d)
    torch.testing.assert_close(r, want, atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,I", [(3, 172), (17, 8192), (1, 5), (5, 1000), (300, 520)])
def test_swiglu(ops, dtype, T, I):
    gu = rnd(T, 2 * I, dtype=dtype, scale=2.0)
    want = torch.nn.functional.silu(gu[:, :I].float()) * gu[:, I:].float()
    torch.testing.assert_close(ops.swiglu(gu).float(), want, **tol(dtype, 1e-5))
    z = torch.zeros(1, 2 * I, dtype=dtype, device=DEV)
    assert ops.swiglu(z).abs().max().item() == 0.0          # silu(0) = 0


# ------------------------------------------------------------------- products
@pytest.mark.parametrize("T,N,K", [(1, 331, 100), (5, 100, 172), (64, 130, 96), (65, 257, 100),
                                   (200, 3072, 2048), (3, 7, 5)])
def test_linear_float32(ops, T, N, K):
    x, w = rnd(T, K, seed=1), rnd(N, K, seed=2, scale=0.05)
    want = (x.double() @ w.double().t()).float()
    torch.testing.assert_close(ops.linear(x, w), want, atol=2e-5, rtol=1e-5)


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("T,N,K", [(1, 2048, 2048), (1, 331, 104), (8, 3072, 2048), (16, 100, 64),
                                   (2, 2048, 8192), (7, 2049, 14336), (3, 128256, 2048), (4, 7, 520),
                                   (17, 130, 96), (33, 8192, 2048), (64, 2048, 8192),
                                   (65, 257, 104), (200, 3072, 2048), (300, 331, 2048),
                                   (128, 128, 64), (5, 100, 100), (70, 100, 172)])
def test_linear_bfloat16(ops, out_dtype, T, N, K):
    """Skinny kernel (T <= 64), matrix-core GEMM (float32 output or forced), library GEMM, and
    the plain kernel for K that is no multiple of 8: all against a float64 product of the same
    bf16-rounded operands."""
    x, w = rnd(T, K, dtype=torch.bfloat16, seed=1), rnd(N, K, dtype=torch.bfloat16, seed=2, scale=0.05)
    want = (x.double() @ w.double().t()).float()
    got = ops.linear(x, w, out_dtype)
    assert got.dtype == out_dtype
    scale = want.abs().max().item()
    if out_dtype == torch.float32:
        torch.testing.assert_close(got, want, atol=2e-5 * max(1.0, scale) * math.sqrt(K / 64), rtol=1e-4)
    else:
        torch.testing.assert_close(got.float(), want, atol=scale / 128, rtol=1e-2)
    old = ops.BF16_GEMM, ops.STREAM_MAX_ROWS
    try:
        ops.BF16_GEMM = "own"
        ops.STREAM_MAX_ROWS = 0                           # the other kernel for few rows
        got2 = ops.linear(x, w, out_dtype)
    finally:
        ops.BF16_GEMM, ops.STREAM_MAX_ROWS = old
    torch.testing.assert_close(got2.float(), got.float(), atol=scale / 128, rtol=1e-2)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16], ids=["f32out", "bf16out"])
@pytest.mark.parametrize("T,N,K", [(1, 2048, 2048), (8, 2048, 8192), (16, 3072, 2048), (3, 130, 96),
                                   (16, 331, 104), (7, 17, 14336), (5, 1001, 4608), (9, 16, 8),
                                   (2, 128256, 256)])
def test_linear_streaming_kernel(ops, out_dtype, T, N, K):
    """The streaming kernel for up to 16 rows (weights through LDS into operand layout), plain and
    gated, against float64 products of the same bf16-rounded operands; sizes that end inside a
    k item, inside a row tile, and with more k items than a workgroup has waves."""
    x, w = rnd(T, K, dtype=torch.bfloat16, seed=3), rnd(N, K, dtype=torch.bfloat16, seed=4, scale=0.05)
    want = (x.double() @ w.double().t()).float()
    old = ops.STREAM_MAX_ROWS
    try:
        ops.STREAM_MAX_ROWS = 16
        if ops.stream_slices(K) > 1:       # one float32 partial result per k slice
            parts = ops.linear(x, w, partials=True)
            assert parts.shape == (ops.stream_slices(K), T, N)
            got = parts.sum(dim=0).to(out_dtype)
        else:
            got = ops.linear(x, w, out_dtype)
        gated = None
        if N % 2 == 0 and out_dtype == torch.bfloat16 and K <= 4096:
            gated = ops.linear_swiglu(x, w)
    finally:
        ops.STREAM_MAX_ROWS = old
    scale = max(1.0, want.abs().max().item())
    if out_dtype == torch.float32:
        torch.testing.assert_close(got, want, atol=2e-5 * scale * math.sqrt(K / 64), rtol=1e-4)
    else:
        torch.testing.assert_close(got.float(), want, atol=scale / 128, rtol=1e-2)
    if gated is not None:
        g, u = want[:, :N // 2].double(), want[:, N // 2:].double()
        want_g = (torch.nn.functional.silu(g) * u).float()
        torch.testing.assert_close(gated.float(), want_g, atol=max(1.0, want_g.abs().max().item()) / 64,
                                   rtol=2e-2)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16], ids=["f32out", "bf16out"])
@pytest.mark.parametrize("T,N,K", [(17, 2048, 2048), (32, 3072, 2048), (31, 2048, 1024), (32, 3072, 3072),
                                   (24, 130, 256), (32, 331, 512), (28, 17, 1792), (20, 16, 768),
                                   (32, 16384, 2048), (19, 1002, 2816), (32, 128256, 256)])
def test_linear_streaming_kernel_for_17_to_32_rows(ops, out_dtype, T, N, K):
    """The streaming kernel's form for 17 to 32 rows (two groups of 16 tokens in a wave's
    registers; k up to 3072 in whole items of 256; two tiles ahead up to eight waves), plain
    and gated, against float64 products of the same bf16-rounded operands: sizes that end inside
    a group of tokens, inside a row tile, with fewer k items than a workgroup has waves; and the
    same rows as the kernel for up to 16 rows gives them (the same sums in the same order)."""
    assert ops.stream_rows(K) >= T
    x, w = rnd(T, K, dtype=torch.bfloat16, seed=3), rnd(N, K, dtype=torch.bfloat16, seed=4, scale=0.05)
    want = (x.double() @ w.double().t()).float()
    got = ops.linear(x, w, out_dtype)
    assert got.dtype == out_dtype and got.shape == (T, N)
    scale = max(1.0, want.abs().max().item())
    if out_dtype == torch.float32:
        torch.testing.assert_close(got, want, atol=2e-5 * scale * math.sqrt(K / 64), rtol=1e-4)
    else:
        torch.testing.assert_close(got.float(), want, atol=scale / 128, rtol=1e-2)
    few = ops.linear(x[:16], w, out_dtype)
    assert torch.equal(got[:16], few)
    old = ops.STREAM_WIDE_MAX_ROWS
    try:
        ops.STREAM_WIDE_MAX_ROWS = 0                       # the library's product instead
        other = ops.linear(x, w, out_dtype)
    finally:
        ops.STREAM_WIDE_MAX_ROWS = old
    torch.testing.assert_close(got.float(), other.float(), atol=scale / 64, rtol=2e-2)
    if N % 2 == 0 and out_dtype == torch.bfloat16:
        gated = ops.linear_swiglu(x, w)
        g, u = want[:, :N // 2].double(), want[:, N // 2:].double()
        want_g = (torch.nn.functional.silu(g) * u).float()
        torch.testing.assert_close(gated.float(), want_g, atol=max(1.0, want_g.abs().max().item()) / 64,
                                   rtol=2e-2)
        assert torch.equal(gated[:16], ops.linear_swiglu(x[:16], w))


@pytest.mark.parametrize("T,H,K,N", [(17, 2048, 2048, 4096), (32, 2048, 2048, 16384), (31, 256, 512, 72),
                                     (32, 1024, 1024, 1002), (25, 768, 2048, 64), (32, 3072, 3072, 512),
                                     (20, 2048, 2816, 3072), (32, 1536, 256, 520)])
@pytest.mark.parametrize("norm_dtype", DTYPES, ids=["normw32", "normw16"])
@pytest.mark.parametrize("round_sum", [True, False])
def test_linear_join_norm_and_linear_scaled_for_17_to_32_rows(ops, T, H, K, N, norm_dtype, round_sum):
    """The norm between two streaming products in two kernels, as above, with 17 to 32 rows:
    against float64 formulas and against the norm kernel on the plain product's result."""
    x = rnd(T, K, dtype=torch.bfloat16, seed=1)
    w1 = rnd(H, K, dtype=torch.bfloat16, seed=2, scale=0.05)
    w2 = rnd(N, H, dtype=torch.bfloat16, seed=3, scale=0.05)
    resid = rnd(T, H, seed=4, scale=3.0)
    nw = (rnd(H, seed=5).abs() + 0.5).to(norm_dtype)
    eps = 1e-5
    product = ops.pending_linear(x, w1, torch.bfloat16)
    assert isinstance(product, ops.PendingProduct) and product.shape == (T, H)
    assert ops.can_join_norm_linear(product, resid, w2)
    delta = x.double() @ w1.double().t()
    if round_sum:
        delta = delta.float().to(torch.bfloat16).double()
    s = resid.double() + delta
    normed = s / torch.sqrt((s * s).mean(-1, keepdim=True) + eps) * nw.double()
    want = normed @ w2.double().t()
    mine = resid.clone()
    xw, ss = ops.linear_join_norm(product, mine, nw, round_sum)
    torch.testing.assert_close(mine.double(), s, atol=2e-2 if round_sum else 1e-3, rtol=1e-2)
    if round_sum:                       # the plain product, rounded, added by the residual kernel
        ref = resid.clone()
        ops.add_residual(ref, product.run(), round_parts=True)
        torch.testing.assert_close(mine, ref, atol=1e-6, rtol=1e-6)
    assert xw.dtype == torch.bfloat16 and xw.shape == (T, H) and ss.shape[0] == -(-T // 16) * 16
    torch.testing.assert_close(ss[:T].sum(1).double(), (mine.double() ** 2).sum(-1), rtol=1e-5, atol=1e-5)
    assert torch.equal(xw, (mine * nw.float()).to(torch.bfloat16))
    for out_dtype in (torch.float32, torch.bfloat16):
        got = ops.linear_scaled(xw, ss, eps, w2, out_dtype)
        assert got.dtype == out_dtype and got.shape == (T, N)
        scale = max(1.0, want.abs().max().item())
        torch.testing.assert_close(got.double(), want, atol=scale / 64, rtol=2e-2)
    # the same rows as 16 rows by themselves give (the first product's sums in the same order;
    # the second's scale from another order of the partial sums of squares)
    few = resid[:16].clone()
    xw16, ss16 = ops.linear_join_norm(ops.pending_linear(x[:16], w1, torch.bfloat16), few, nw, round_sum)
    assert torch.equal(few, mine[:16]) and torch.equal(xw16, xw[:16])
    torch.testing.assert_close(ops.linear_scaled(xw16, ss16, eps, w2, torch.float32),
                               ops.linear_scaled(xw, ss, eps, w2, torch.float32)[:16], atol=1e-4, rtol=1e-5)
    if N % 2 == 0:
        got = ops.linear_scaled(xw, ss, eps, w2, torch.bfloat16, gated=True)
        g, u = want[:, :N // 2], want[:, N // 2:]
        want_g = torch.nn.functional.silu(g) * u
        torch.testing.assert_close(got.double(), want_g, atol=max(1.0, want_g.abs().max().item()) / 32,
                                   rtol=3e-2)
    # a k that no wave holds 17 rows of, or more than 32 rows: the plain product comes back
    assert isinstance(ops.pending_linear(rnd(T, 4096, dtype=torch.bfloat16), rnd(64, 4096, dtype=torch.bfloat16)),
                      torch.Tensor)
    assert isinstance(ops.pending_linear(rnd(33, K, dtype=torch.bfloat16), w1), torch.Tensor)


@pytest.mark.parametrize("T,N,K", [(17, 2048, 2048), (64, 2048, 8192), (33, 3072, 2048), (24, 130, 96),
                                   (64, 331, 104), (48, 17, 14336), (19, 1001, 4608), (40, 16, 8),
                                   (64, 4096, 14336), (50, 3072, 3072), (64, 3072, 8192),
                                   (32, 4096, 14344), (48, 8192, 3000), (17, 6144, 1536)])
def test_linear_split_k_kernel(ops, monkeypatch, T, N, K):
    """The split-k kernel that 17 to 64 rows take where the result joins the residual stream:
    float32 partial sums per k slice against float64 products of the same bf16-rounded
    operands; sizes that end inside a slice, inside a block of weight rows and inside a token
    group.  A row's sums are the same bits with 17 rows in the call as with 64.  (With the
    streaming kernel's form for 17 to 64 rows switched off, which takes the short k first.)"""
    monkeypatch.setattr(ops, "STREAM_WIDE_MAX_ROWS", 0)
    x, w = rnd(T, K, dtype=torch.bfloat16, seed=3), rnd(N, K, dtype=torch.bfloat16, seed=4, scale=0.05)
    want = (x.double() @ w.double().t()).float()
    parts = ops.linear(x, w, partials=True)
    assert parts.dim() == 3 and parts.shape[1:] == (T, N) and parts.dtype == torch.float32
    # pieces of 512 k (256 where the product is small), one or two of them per workgroup
    groups, pieces = -(-N // 64), -(-K // 512)
    per_group = 2 if groups * pieces > 512 else 1
    assert parts.shape[0] == (-(-K // 256) if groups * pieces < 256 else -(-K // (512 * per_group)))
    got = parts.sum(dim=0)
    scale = max(1.0, want.abs().max().item())
    torch.testing.assert_close(got, want, atol=2e-5 * scale * math.sqrt(K / 64), rtol=1e-4)
    fewer = ops.linear(x[:17].contiguous(), w, partials=True)
    assert torch.equal(fewer, parts[:, :17])
    # the residual stream's consumers add the slices in order and round once
    resid = rnd(T, N, seed=5)
    summed = resid.clone()
    ops.add_residual(summed, parts, round_parts=True)
    rounded = parts[0].clone()
    for s in range(1, parts.shape[0]):
        rounded += parts[s]
    assert torch.equal(summed, resid + rounded.to(torch.bfloat16).float())


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16], ids=["f32out", "bf16out"])
@pytest.mark.parametrize("T,N,K", [(17, 3072, 2048), (64, 16384, 2048), (100, 2048, 8192), (575, 5120, 3072),
                                   (2048, 2048, 2048), (33, 331, 104), (300, 1001, 776), (65, 8, 8)])
def test_library_product_called_directly(ops, monkeypatch, out_dtype, T, N, K):
    """bfloat16 products beyond the hand-written kernels' row counts go to hipBLASLt through its
    own entry points: against float64 products of the same operands, against the same library
    through torch.matmul, strided operands, and twice (the second call takes the kept plan)."""
    monkeypatch.setattr(ops, "STREAM_WIDE_MAX_ROWS", 0)   # 17 to 64 rows of a short k: the library's too
    from rust_llm_inference_server_amd.ops import lib
    assert lib.library_workspace(torch.device(DEV)) is not None, "hipBLASLt's entry points were not found"
    x, w = rnd(T, K, dtype=torch.bfloat16, seed=3), rnd(N, K, dtype=torch.bfloat16, seed=4, scale=0.05)
    want = (x.double() @ w.double().t()).float()
    scale = max(1.0, want.abs().max().item())
    tol_ = dict(atol=(2e-5 if out_dtype == torch.float32 else 8e-3) * scale * math.sqrt(K / 64), rtol=1e-2)
    old = ops.LIBRARY_GEMM_DIRECT
    try:
        ops.LIBRARY_GEMM_DIRECT = False
        through_torch = ops.linear(x, w, out_dtype)
        ops.LIBRARY_GEMM_DIRECT = True
        for _ in range(2):
            got = ops.linear(x, w, out_dtype)
            assert got.dtype == out_dtype and got.shape == (T, N)
            torch.testing.assert_close(got.float(), want, **tol_)
            torch.testing.assert_close(got.float(), through_torch.float(), **tol_)
        # rows of x and of the weight inside wider arrays
        wide_x = rnd(T, K + 24, dtype=torch.bfloat16, seed=5)
        wide_w = rnd(N, K + 8, dtype=torch.bfloat16, seed=6, scale=0.05)
        got = ops.linear(wide_x[:, 8:8 + K], wide_w[:, :K], out_dtype)
        want = (wide_x[:, 8:8 + K].double() @ wide_w[:, :K].double().t()).float()
        torch.testing.assert_close(got.float(), want, **tol_)
    finally:
        ops.LIBRARY_GEMM_DIRECT = old


def test_library_products_are_tried_out_before_their_first_use(ops, monkeypatch):
    """A shape of the library's products (33 to 64 rows, or a multiple of 32 up to 1,024) is
    tried out before its first product: the heuristics' first candidates are timed over the
    weights of that shape in turn and the fastest is kept.  Once, and never under a capturing
    stream: a shape keeps its algorithm, so a product gives the same bits every time; other row
    counts, and everything with the switch off, take the heuristics' first choice untimed.
    (Shapes that nothing else in the tests uses: a plan made earlier would not be tried out.)"""
    monkeypatch.setattr(ops, "STREAM_WIDE_MAX_ROWS", 0)
    N, K = 1192, 1096
    ws = [rnd(N, K, dtype=torch.bfloat16, seed=20 + i, scale=0.05) for i in range(3)]
    ops.note_weights(ws + [rnd(N, K, seed=9), rnd(8, dtype=torch.bfloat16, seed=9)])   # (skipped)
    log = ops.tune_log

    def product(T, out_dtype=torch.bfloat16, w=ws[0], **kw):
        x = rnd(T, K, dtype=torch.bfloat16, seed=T)
        got = ops.linear(x, w, out_dtype, **kw)
        want = (x.double() @ w.double().t()).float()
        scale = max(1.0, want.abs().max().item())
        torch.testing.assert_close(got.float() if got.dim() == 2 else got.sum(0), want,
                                   atol=8e-3 * scale * math.sqrt(K / 64), rtol=1e-2)
        return got

    before = len(log)
    first = product(96)
    assert len(log) == before + 1
    T, n, k, slices, taken, us_first, us_taken = log[-1]
    assert (T, n, k, slices) == (96, N, K, 1) and 0 <= taken < ops.LIBRARY_TUNE_CANDIDATES
    assert 0 < us_taken <= us_first and (taken == 0 or us_taken < us_first * (1 - ops.LIBRARY_TUNE_MARGIN))
    assert torch.equal(product(96), first) and len(log) == before + 1        # once
    assert torch.equal(product(96, w=ws[1]), ops.linear(rnd(96, K, dtype=torch.bfloat16, seed=96), ws[1],
                                                        torch.bfloat16)) and len(log) == before + 1
    product(40)                                  # a decode batch of 33 to 64 requests
    product(64, torch.float32)                   # ... another output type is another shape
    assert len(log) == before + 3
    # beyond 64 rows multiples of 32 are tried out; a count in between takes the algorithm of
    # the next multiple (which is tried out for it, on rows of nothing), untimed
    adopted = len(ops.adopt_log)
    product(100)
    assert len(log) == before + 4 and log[-1][0] == 128
    assert len(ops.adopt_log) == adopted + 1 and ops.adopt_log[-1][:5] == (100, 128, N, K, 1)
    assert -1 <= ops.adopt_log[-1][5] < 16
    product(128)                                 # (has its plan from that)
    product(101)
    assert len(log) == before + 4 and len(ops.adopt_log) == adopted + 2
    product(1056)                                # nothing beyond 1,024 rows
    assert len(log) == before + 4 and len(ops.adopt_log) == adopted + 2
    monkeypatch.setattr(ops, "LIBRARY_TUNE_ROWS", {200})      # a named count (an engine's budget)
    product(200)
    monkeypatch.setattr(ops, "LIBRARY_TUNE_ROWS", set())
    assert len(log) == before + 5 and log[-1][0] == 200 and len(ops.adopt_log) == adopted + 2
    monkeypatch.setattr(ops, "LIBRARY_TUNE", False)
    product(256)
    assert len(log) == before + 5
    monkeypatch.setattr(ops, "LIBRARY_TUNE", True)
    product(256)                                 # (has a plan by now: nothing is tried out)
    assert len(log) == before + 5 and len(ops.adopt_log) == adopted + 2
    before += 2
    # under a capturing stream nothing can be timed: the shape takes the heuristics' first
    x = rnd(160, K, dtype=torch.bfloat16, seed=160)
    from rust_llm_inference_server_amd.ops import lib
    graph = torch.cuda.CUDAGraph()
    with lib.workspace_owner(torch.cuda.current_stream()), torch.cuda.graph(graph):
        captured = ops.linear(x, ws[2], torch.bfloat16)
    graph.replay()
    torch.cuda.synchronize()
    assert len(log) == before + 3
    assert torch.equal(captured, ops.linear(x, ws[2], torch.bfloat16)) and len(log) == before + 3


@pytest.mark.parametrize("T,N,K", [(100, 2048, 8192), (512, 3072, 8192), (300, 136, 14336), (1024, 264, 8192),
                                   (65, 8, 8192)])
def test_library_product_in_slices_of_k(ops, T, N, K):
    """A product over a long k whose consumer takes partial sums goes to the library as one
    batched call over slices of k, at the row counts of a budgeted step: the stack's slices
    against float64 products over the same slice, their sum against the whole product, rows of
    the operands inside wider arrays, twice (the kept plan); and the rule for the slices."""
    from rust_llm_inference_server_amd.ops import lib
    assert lib.library_workspace(torch.device(DEV)) is not None, "hipBLASLt's entry points were not found"
    assert ops.library_slices(64, 8192) == 1 and ops.library_slices(2048, 8192) == 2
    assert ops.library_slices(1025, 14336) == 2 and ops.library_slices(2049, 8192) == 1
    assert ops.library_slices(512, 4096) == 1 and ops.library_slices(512, 8192 + 8) == 1
    assert ops.library_slices(512, 8192) == 4 and ops.library_slices(256, 8192) == 8
    assert ops.library_slices(300, 14336) == 4 and ops.library_slices(100, 14336) == 8
    assert ops.library_slices(300, 8192 + 16) == 2 and ops.library_slices(100, 8192 + 32) == 4
    slices = ops.library_slices(T, K)
    assert slices > 1
    wide_x = rnd(T, K + 24, dtype=torch.bfloat16, seed=5)
    wide_w = rnd(N, K + 8, dtype=torch.bfloat16, seed=6, scale=0.05)
    for x, w in ((wide_x[:, :K].contiguous(), wide_w[:, :K].contiguous()), (wide_x[:, 8:8 + K], wide_w[:, :K])):
        for _ in range(2):
            got = ops.linear(x, w, torch.bfloat16, partials=True)
            assert got.dtype == torch.float32 and got.shape == (slices, T, N)
            step = K // slices
            for s in range(slices):
                want = (x[:, s * step:(s + 1) * step].double() @ w[:, s * step:(s + 1) * step].double().t()).float()
                scale = max(1.0, want.abs().max().item())
                torch.testing.assert_close(got[s], want, atol=2e-5 * scale * math.sqrt(step / 64), rtol=1e-2)
            whole = ops.linear(x, w, torch.float32)
            torch.testing.assert_close(got.sum(0), whole, atol=1e-3, rtol=1e-3)


@pytest.mark.parametrize("T,N,K,parts,rows", [(1, 2048, 2048, 0, False), (8, 3072, 2048, 1, False),
                                              (16, 344, 104, 2, False), (5, 1001, 4096, 1, False),
                                              (3, 128256, 256, 1, True), (7, 64, 776, 3, True),
                                              (8, 16384, 2048, 1, False)])
@pytest.mark.parametrize("norm_dtype", DTYPES, ids=["normw32", "normw16"])
def test_norm_linear(ops, T, N, K, parts, rows, norm_dtype):
    """RMSNorm fused into the streaming product, plain and gated, float32 and bfloat16 output:
    no delta, a bfloat16 delta, float32 partial sums; a row selection; the summed residual that
    comes back.  Against float64 formulas; the norm weight is far from one so that leaving it
    out, or applying it after the product, would show."""
    total = T + 5 if rows else T
    resid = rnd(total, K, seed=1, scale=3.0)
    if parts == 0:
        delta = None
    elif parts == 1:
        delta = rnd(total, K, dtype=torch.bfloat16, seed=2)
    else:
        delta = rnd(parts, total, K, seed=2)
    nw = (rnd(K, seed=3).abs() + 0.5).to(norm_dtype)
    w = rnd(N, K, dtype=torch.bfloat16, seed=4, scale=0.05)
    sel = torch.tensor([(3 * i + 1) % total for i in range(T)], dtype=torch.int32, device=DEV) if rows else None
    eps = 1e-5
    s = resid.double()
    if delta is not None:
        s = s + (delta.double() if parts == 1 else delta.double().sum(0))
    src = s if sel is None else s[sel.long()]
    normed = src / torch.sqrt((src * src).mean(-1, keepdim=True) + eps) * nw.double()
    want = normed @ w.double().t()
    assert ops.can_fuse_norm_linear(resid, w, T)
    resid_before = resid.clone()
    for out_dtype in (torch.float32, torch.bfloat16):
        got, total_out = ops.norm_linear(resid, delta, nw, eps, w, out_dtype, rows=sel)
        assert got.dtype == out_dtype and got.shape == (T, N)
        scale = max(1.0, want.abs().max().item())
        torch.testing.assert_close(got.double(), want, atol=scale / 64, rtol=2e-2)
        assert torch.equal(resid, resid_before)              # the input residual is left alone
        if sel is not None:
            assert total_out is None
        elif delta is None:
            assert total_out is resid
        else:
            torch.testing.assert_close(total_out.double(), s, atol=1e-5, rtol=1e-6)
    if N % 2 == 0:
        got, _ = ops.norm_linear(resid, delta, nw, eps, w, torch.bfloat16, gated=True, rows=sel)
        g, u = want[:, :N // 2], want[:, N // 2:]
        want_g = torch.nn.functional.silu(g) * u
        torch.testing.assert_close(got.double(), want_g, atol=max(1.0, want_g.abs().max().item()) / 32,
                                   rtol=3e-2)


@pytest.mark.parametrize("T,H,K,N", [(1, 2048, 2048, 4096), (8, 2048, 2048, 16384), (16, 104, 344, 72),
                                     (5, 4096, 1000, 1002), (7, 776, 4096, 64), (13, 3072, 3072, 512),
                                     (8, 3072, 2048, 3072), (16, 2560, 3072, 520), (3, 4088, 4096, 72),
                                     (8, 2048, 8192, 3072), (16, 3072, 8192, 520), (3, 1000, 5120, 72),
                                     (1, 2048, 6144, 64)])
@pytest.mark.parametrize("norm_dtype", DTYPES, ids=["normw32", "normw16"])
@pytest.mark.parametrize("round_sum", [True, False])
def test_linear_join_norm_and_linear_scaled(ops, T, H, K, N, norm_dtype, round_sum):
    """A norm between two streaming products in two kernels with no pass over whole rows: the
    first adds x @ w1.T to the residual (rounded to bfloat16 first, or not), in place, and
    leaves the rows times the norm's weight and their sums of squares per tile of columns; the
    second multiplies those rows by w2 and scales by the rsqrt of the mean square, plain and
    gated.  Against float64 formulas, and against the one-kernel norm in front of the second
    product fed with the first product's result (the same roundings, another order of the sums
    of squares).  Tiles of 8, 12 and 16 weight rows; first products over a feed-forward's width
    (4096 < K <= 8192 in whole fours of k items) take four items per wave."""
    x = rnd(T, K, dtype=torch.bfloat16, seed=1)
    w1 = rnd(H, K, dtype=torch.bfloat16, seed=2, scale=0.05)
    w2 = rnd(N, H, dtype=torch.bfloat16, seed=3, scale=0.05)
    resid = rnd(T, H, seed=4, scale=3.0)
    nw = (rnd(H, seed=5).abs() + 0.5).to(norm_dtype)
    eps = 1e-5
    product = ops.pending_linear(x, w1, torch.bfloat16)
    assert isinstance(product, ops.PendingProduct) and product.shape == (T, H)
    assert ops.can_join_norm_linear(product, resid, w2)
    delta = x.double() @ w1.double().t()
    if round_sum:
        delta = delta.float().to(torch.bfloat16).double()
    s = resid.double() + delta
    normed = s / torch.sqrt((s * s).mean(-1, keepdim=True) + eps) * nw.double()
    want = normed @ w2.double().t()
    # the one-kernel norm on the plain product's result
    ref_y, ref_total = ops.norm_linear(resid, product.run() if round_sum else
                                       ops.linear(x, w1, torch.float32).unsqueeze(0),
                                       nw, eps, w2, torch.float32, round_parts=round_sum)
    mine = resid.clone()
    xw, ss = ops.linear_join_norm(product, mine, nw, round_sum)
    torch.testing.assert_close(mine.double(), s, atol=2e-2 if round_sum else 1e-3, rtol=1e-2)
    torch.testing.assert_close(mine, ref_total, atol=1e-6 if round_sum else 1e-4, rtol=1e-6)
    assert xw.dtype == torch.bfloat16 and xw.shape == (T, H) and ss.shape[0] == 16
    torch.testing.assert_close(ss[:T].sum(1).double(), (mine.double() ** 2).sum(-1), rtol=1e-5, atol=1e-5)
    assert torch.equal(xw, (mine * nw.float()).to(torch.bfloat16))
    for out_dtype in (torch.float32, torch.bfloat16):
        got = ops.linear_scaled(xw, ss, eps, w2, out_dtype)
        assert got.dtype == out_dtype and got.shape == (T, N)
        scale = max(1.0, want.abs().max().item())
        torch.testing.assert_close(got.double(), want, atol=scale / 64, rtol=2e-2)
    got = ops.linear_scaled(xw, ss, eps, w2, torch.float32)
    torch.testing.assert_close(got, ref_y, atol=max(1.0, want.abs().max().item()) * 1e-4, rtol=1e-4)
    if N % 2 == 0:
        got = ops.linear_scaled(xw, ss, eps, w2, torch.bfloat16, gated=True)
        g, u = want[:, :N // 2], want[:, N // 2:]
        want_g = torch.nn.functional.silu(g) * u
        torch.testing.assert_close(got.double(), want_g, atol=max(1.0, want_g.abs().max().item()) / 32,
                                   rtol=3e-2)
    # more than one k slice, more than 32 rows (more than 16 of a long k), or float32: the plain
    # product comes back
    assert isinstance(ops.pending_linear(rnd(T, 8448, dtype=torch.bfloat16), rnd(64, 8448, dtype=torch.bfloat16)),
                      torch.Tensor)
    assert isinstance(ops.pending_linear(rnd(33, K, dtype=torch.bfloat16), w1), torch.Tensor)
    assert isinstance(ops.pending_linear(rnd(17, 8192, dtype=torch.bfloat16), rnd(64, 8192, dtype=torch.bfloat16)),
                      torch.Tensor)
    assert isinstance(ops.pending_linear(rnd(T, K), rnd(H, K)), torch.Tensor)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,I,K", [(1, 8192, 2048), (8, 172, 104), (16, 320, 192), (33, 1000, 256),
                                   (8, 8192, 2048), (3, 1001, 4608), (8, 77, 14336),
                                   (64, 8192, 2048), (65, 172, 104), (5, 100, 100)])
def test_linear_swiglu(ops, dtype, T, I, K):
    """The gated product (one kernel up to 64 bfloat16 rows, two kernels otherwise) against
    silu(x Wg^T) * (x Wu^T) in float64."""
    x = rnd(T, K, dtype=dtype, seed=1)
    w = rnd(2 * I, K, dtype=dtype, seed=2, scale=0.05)
    g = x.double() @ w[:I].double().t()
    u = x.double() @ w[I:].double().t()
    want = (torch.nn.functional.silu(g) * u).float()
    got = ops.linear_swiglu(x, w)
    assert got.dtype == dtype and got.shape == (T, I)
    old = ops.STREAM_MAX_ROWS, ops.BF16_GEMM
    try:
        ops.STREAM_MAX_ROWS, ops.BF16_GEMM = 0, "own"         # the skinny kernel up to 64 rows
        other = ops.linear_swiglu(x, w)
    finally:
        ops.STREAM_MAX_ROWS, ops.BF16_GEMM = old
    torch.testing.assert_close(other.float(), got.float(), atol=0.05, rtol=2e-2)
    scale = max(1.0, want.abs().max().item())
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, atol=1e-4 * scale, rtol=1e-4)
    else:
        torch.testing.assert_close(got.float(), want, atol=scale / 64, rtol=2e-2)


def test_linear_mixed_dtypes(ops):
    # a weight stored in 32 bits stays so: bfloat16 activations times a float32 weight
    x, w = rnd(9, 100, dtype=torch.bfloat16, seed=1), rnd(50, 100, seed=2)
    want = x.float() @ w.t()
    torch.testing.assert_close(ops.linear(x, w, torch.bfloat16).float(), want, atol=0.1, rtol=1e-2)
    torch.testing.assert_close(ops.linear(x, w, torch.float32), want, atol=1e-4, rtol=1e-4)


def test_linear_rows_do_not_depend_on_the_batch(ops):
    """A row's product is the same bits whichever other rows share the call, within the row
    counts that one of the engine's kernels takes (float32: any; bfloat16: up to 16 rows and 17
    to 32 rows; beyond that the library computes, which promises no such thing)."""
    for dtype, counts in ((torch.float32, (40, 16)), (torch.bfloat16, (30, 16))):
        for rows in counts:
            lo, hi = (5, 23) if rows > 16 else (3, 9)
            x, w = rnd(rows, 256, dtype=dtype, seed=1), rnd(300, 256, dtype=dtype, seed=2)
            full = ops.linear(x, w, torch.float32)
            part = ops.linear(x[lo:hi].contiguous(), w, torch.float32)
            torch.testing.assert_close(part, full[lo:hi], atol=0, rtol=0)


# ---------------------------------------------------------- rotation + cache write
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T", [11, 77])
@pytest.mark.parametrize("nh,nkv,d,rot,ps", [(4, 1, 16, 16, 16), (6, 2, 32, 32, 8), (5, 5, 48, 48, 16),
                                              (3, 1, 80, 40, 32), (32, 8, 64, 64, 16), (2, 2, 80, 48, 16),
                                              (16, 8, 256, 256, 16), (3, 3, 24, 0, 8)])
def test_rope_kv_write(ops, dtype, T, nh, nkv, d, rot, ps):
    """Scattered slots (T = 11) and runs of adjacent slots that start in the middle of a page,
    with tokens that are not stored (slot -1) among them (T = 77)."""
    g = torch.Generator().manual_seed(T)
    positions = torch.randint(0, 128, (T,), generator=g, dtype=torch.int32)
    positions[:3] = torch.tensor([0, 1, 127])
    if rot:
        inv = plain.inv_freqs(rot, 10000.0, None)
        cos_all, sin_all = plain.rope_tables(inv, range(128))
    else:
        cos_all = sin_all = None
    qkv = rnd(T, (nh + 2 * nkv) * d, dtype=dtype, seed=4)
    if T == 11:
        pages = 9
        slots = torch.randperm(pages * ps, generator=g)[:T].to(torch.int32)
    else:
        pages = (3 * ps + 64 + 37) // ps + 2
        slots = torch.cat([torch.arange(5, 5 + 40), torch.arange(3 * ps + 64, 3 * ps + 64 + 37)]).to(torch.int32)
        slots[[7, 50, 76]] = -1
    k_pages = torch.zeros(pages, nkv, ps, d, dtype=dtype, device=DEV)
    v_pages = torch.zeros(pages, nkv, d, ps, dtype=dtype, device=DEV)
    src = qkv.clone()
    ops.rope_kv_write(qkv, nh, nkv, d, None if cos_all is None else cos_all.to(DEV),
                      None if sin_all is None else sin_all.to(DEV), positions.to(DEV),
                      slots.to(DEV), k_pages, v_pages, ps)
    x = src.float().cpu()
    q = x[:, :nh * d].reshape(T, nh, d)
    k = x[:, nh * d:(nh + nkv) * d].reshape(T, nkv, d)
    v = x[:, (nh + nkv) * d:].reshape(T, nkv, d)

    def rotate(t):          # (T, heads, d): rotate the first `rot` dims, pass the rest
        if not rot:
            return t
        cos, sin = cos_all[positions.long()], sin_all[positions.long()]
        r = plain.rope_apply(t[..., :rot].transpose(0, 1), cos, sin).transpose(0, 1)
        return torch.cat([r, t[..., rot:]], dim=-1)

    t = tol(dtype, 1e-5, 1e-2)
    torch.testing.assert_close(qkv[:, :nh * d].float().cpu().reshape(T, nh, d), rotate(q), **t)
    torch.testing.assert_close(qkv[:, nh * d:].cpu(), src[:, nh * d:].cpu(), atol=0, rtol=0)
    kr = rotate(k)
    kp, vp = k_pages.float().cpu(), v_pages.float().cpu()
    for i in range(T):
        if int(slots[i]) < 0:
            continue
        page, off = int(slots[i]) // ps, int(slots[i]) % ps
        torch.testing.assert_close(kp[page, :, off, :], kr[i], **t)
        torch.testing.assert_close(vp[page, :, :, off], v[i], atol=0, rtol=0)
    # rows that were not written stay zero
    written = torch.zeros(pages * ps, dtype=torch.bool)
    written[slots[slots >= 0].long()] = True
    k_rows = kp.abs().sum(dim=3).transpose(1, 2).reshape(pages * ps, nkv)
    v_rows = vp.abs().sum(dim=2).transpose(1, 2).reshape(pages * ps, nkv)
    assert k_rows[~written].max().item() == 0.0 and v_rows[~written].max().item() == 0.0


def test_rope_position_zero_is_identity_and_norm_is_kept(ops):
    nh, nkv, d, ps = 2, 1, 32, 8
    inv = plain.inv_freqs(d, 10000.0, None)
    cos, sin = plain.rope_tables(inv, range(64))
    qkv = rnd(2, (nh + 2 * nkv) * d, seed=3)
    src = qkv.clone()
    pos = torch.tensor([0, 37], dtype=torch.int32, device=DEV)
    ops.rope_kv_write(qkv, nh, nkv, d, cos.to(DEV), sin.to(DEV), pos, None, None, None, ps,
                      write_kv=False)
    torch.testing.assert_close(qkv[0], src[0], atol=0, rtol=0)
    n0 = src[1, :nh * d].reshape(nh, d).norm(dim=-1)
    n1 = qkv[1, :nh * d].reshape(nh, d).norm(dim=-1)
    torch.testing.assert_close(n0, n1, atol=1e-5, rtol=1e-5)
    assert (qkv[1, :nh * d] - src[1, :nh * d]).abs().max().item() > 0.1


# ---------------------------------------------------------------------- attention
class FakeStep:
    pass


@contextlib.contextmanager
def attention_constants(**values):
    """Run with other constants in the attention planner (partition sizes, tile forms, key
    runs): every combination must give the same numbers up to rounding."""
    from rust_llm_inference_server_amd.ops import attention_plan as ap
    old = {k: getattr(ap, k) for k in values}
    try:
        for k, v in values.items():
            setattr(ap, k, v)
        yield
    finally:
        for k, v in old.items():
            setattr(ap, k, v)


def key_runs(n):
    """Constants that cut every multi-token sequence's tiles into n runs where it has the keys."""
    return dict(PREFILL_SPLIT_UNITS=1 << 20, PREFILL_SPLIT_MIN_KEYS=1, PREFILL_MAX_RUNS=n)


# partitions of the decode kernels: (keys per partition, most partitions)
DECODE_CUTS = [(1024, 16), (256, 16), (256, 2)]


def paged_case(lens_cached, lens_new, nh, nkv, d, ps, dtype, seed=0, q_scale=1.0):
    """A batch of sequences with scattered pages.  Returns (qkv, k_pages, v_pages, tables,
    step, per-sequence K and V in float32, q in float32)."""
    S = len(lens_new)
    g = torch.Generator().manual_seed(seed)
    totals = [c + n for c, n in zip(lens_cached, lens_new)]
    pages_per = [-(-t // ps) for t in totals]
    num_pages = sum(pages_per) + 3
    perm = torch.randperm(num_pages, generator=g).tolist()
    tables, it = [], iter(perm)
    for p in pages_per:
        tables.append([next(it) for _ in range(p)])
    width = max(8, max(pages_per))
    bt = torch.zeros(S, width, dtype=torch.int32)
    for s, t in enumerate(tables):
        bt[s, :len(t)] = torch.tensor(t, dtype=torch.int32)
    k_pages = torch.randn(num_pages, nkv, ps, d, generator=g).to(dtype)   # stale contents
    v_pages = torch.randn(num_pages, nkv, d, ps, generator=g).to(dtype)
    ks, vs = [], []
    for s in range(S):
        k = torch.randn(totals[s], nkv, d, generator=g).to(dtype)
        v = torch.randn(totals[s], nkv, d, generator=g).to(dtype)
        for p in range(totals[s]):
            k_pages[tables[s][p // ps], :, p % ps, :] = k[p]
            v_pages[tables[s][p // ps], :, :, p % ps] = v[p]
        ks.append(k.float())
        vs.append(v.float())
    T = sum(lens_new)
    qkv = (torch.randn(T, (nh + 2 * nkv) * d, generator=g) * q_scale).to(dtype)
    step = FakeStep()
    step.num_tokens, step.num_seqs = T, S
    cu = [0]
    for n in lens_new:
        cu.append(cu[-1] + n)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    step.cu_seqlens, step.start_pos = i32(cu), i32(lens_cached)
    step.ctx_lens = i32(totals)
    step.positions = i32([c + i for c, n in zip(lens_cached, lens_new) for i in range(n)])
    step.seq_of_token = i32([s for s, n in enumerate(lens_new) for _ in range(n)])
    step.max_context, step.max_new = max(totals), max(lens_new)
    step.all_decode = all(n == 1 for n in lens_new)
    # single tokens that lead the batch, as the engine's steps order them (the kernels' work
    # lists are planned from these host lengths at the call)
    lead = next((i for i, n in enumerate(lens_new) if n != 1), S)
    if not all(n > 1 for n in lens_new[lead:]):
        lead = 0
    step.num_single = lead
    step.lengths = StepLengths(np.asarray(lens_cached, dtype=np.int64),
                               np.asarray(lens_new, dtype=np.int64), lead, ps)
    return (qkv.to(DEV), k_pages.to(DEV), v_pages.to(DEV), bt.to(DEV), step, ks, vs, cu)


def reference_attention(qkv, ks, vs, cu, lens_cached, lens_new, nh, nkv, d, scale, window):
    outs = []
    q_all = qkv.float().cpu()[:, :nh * d]
    for s, (c, n) in enumerate(zip(lens_cached, lens_new)):
        q = q_all[cu[s]:cu[s + 1]].reshape(n, nh, d).transpose(0, 1)
        k, v = ks[s].transpose(0, 1), vs[s].transpose(0, 1)
        mask = plain.causal_mask(n, c, window)
        o = plain.gqa_attention(q, k, v, mask, scale)
        outs.append(o.transpose(0, 1).reshape(n, nh * d))
    return torch.cat(outs)


LAYOUTS = [(4, 1, 16, 16), (6, 2, 32, 8), (5, 5, 48, 16), (32, 8, 64, 16), (24, 8, 128, 16),
           (8, 8, 64, 32), (12, 2, 128, 64), (3, 1, 80, 8), (16, 2, 256, 16), (9, 3, 112, 16)]


def kinds_and_dtypes(*kinds):
    """Every kernel family with the dtypes it takes: the matrix-core prefill kernel is
    bfloat16 only."""
    return [pytest.param(k, dt, id=f"{k}-{str(dt).split('.')[-1]}") for k in kinds for dt in DTYPES
            if k != "prefill" or dt == torch.bfloat16]


@pytest.mark.parametrize("nh,nkv,d,ps", LAYOUTS)
@pytest.mark.parametrize("kind,dtype", kinds_and_dtypes("generic", "prefill"))
def test_attention_mixed_batch(ops, dtype, nh, nkv, d, ps, kind):
    """Portions of prompts (with and without cached positions, across page and tile edges)
    beside single tokens, in one batch, through scattered block tables."""
    cached = [0, 5, 40, 0, 63, 130, 17]
    new = [33, 1, 70, 2, 1, 129, 64]
    scale = 1.0 / math.sqrt(d)
    qkv, kp, vp, bt, step, ks, vs, cu = paged_case(cached, new, nh, nkv, d, ps, dtype, seed=nh)
    got = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, None, force=kind)
    want = reference_attention(qkv, ks, vs, cu, cached, new, nh, nkv, d, scale, None)
    torch.testing.assert_close(got.float().cpu(), want, **tol(dtype, 2e-5, 2e-2))


@pytest.mark.parametrize("nh,nkv,d,ps", [(32, 8, 64, 16), (24, 8, 128, 16), (6, 2, 32, 8), (5, 5, 48, 16),
                                         (34, 2, 16, 16)])
@pytest.mark.parametrize("window", [None, 70])
def test_attention_single_tokens_beside_portions(ops, nh, nkv, d, ps, window):
    """Single tokens that lead a batch of portions take the decode kernel, the portions the
    prefill kernel: same result as the plain implementation, and as the prefill kernel alone.
    17 query heads per KV head are more than the decode kernel takes: then nothing is split."""
    dtype = torch.bfloat16
    cached = [5, 63, 300, 1000, 0, 40, 0, 130, 17]
    new = [1, 1, 1, 1, 33, 70, 2, 129, 64]
    scale = 1.0 / math.sqrt(d)
    qkv, kp, vp, bt, step, ks, vs, cu = paged_case(cached, new, nh, nkv, d, ps, dtype, seed=nh + 1)
    assert step.num_single == 4
    want = reference_attention(qkv, ks, vs, cu, cached, new, nh, nkv, d, scale, window)
    got = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, window)
    torch.testing.assert_close(got.float().cpu(), want, **tol(dtype, 2e-5, 2e-2))
    whole = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, window, force="prefill")
    torch.testing.assert_close(got.float(), whole.float(), atol=2e-2, rtol=2e-2)
    assert torch.equal(got[4:], whole[4:])                 # the portions' rows: same kernel, same tiles
    old = ops.SPLIT_MIXED_ATTENTION
    try:
        ops.SPLIT_MIXED_ATTENTION = False
        assert torch.equal(ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, window), whole)
    finally:
        ops.SPLIT_MIXED_ATTENTION = old


@pytest.mark.parametrize("nh,nkv,d,ps", [(32, 8, 64, 16), (24, 8, 128, 16), (6, 2, 32, 8), (5, 5, 48, 16),
                                         (3, 1, 96, 32), (9, 3, 112, 16), (4, 2, 256, 16)])
@pytest.mark.parametrize("window", [None, 70, 200])
def test_attention_prefill_tiles_of_128_queries(ops, nh, nkv, d, ps, window):
    """The prefill kernel with two query blocks per wave (tiles of 128 new tokens, which long
    prompts take) against the plain implementation and against its 64-token form: portions that
    end inside a tile, inside a query block, with and without cached positions, single tokens
    among them.  Head sizes beyond 128 keep the 64-token form."""
    dtype = torch.bfloat16
    cached = [0, 5, 40, 0, 63, 130, 17, 300]
    new = [33, 1, 70, 2, 129, 257, 128, 200]
    scale = 1.0 / math.sqrt(d)
    qkv, kp, vp, bt, step, ks, vs, cu = paged_case(cached, new, nh, nkv, d, ps, dtype, seed=nh + 2)
    want = reference_attention(qkv, ks, vs, cu, cached, new, nh, nkv, d, scale, window)
    narrow = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, window)
    with attention_constants(PREFILL_WIDE_MIN_GROUPS=0):
        got = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, window)
    torch.testing.assert_close(got.float().cpu(), want, **tol(dtype, 2e-5, 2e-2))
    torch.testing.assert_close(got.float(), narrow.float(), atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("nh,nkv,d,ps", [(32, 8, 64, 16), (24, 8, 128, 16), (6, 2, 32, 8), (3, 1, 96, 32),
                                         (4, 2, 256, 16)])
@pytest.mark.parametrize("window", [None, 70])
@pytest.mark.parametrize("splits", [2, 3, 7])
def test_attention_prefill_with_keys_cut_into_runs(ops, nh, nkv, d, ps, window, splits):
    """The prefill kernel with every tile's keys cut into runs that separate workgroups take and
    a merge afterwards (what a portion of a long prompt gets): against the plain
    implementation, with both tile sizes; runs without keys, queries that see no key of a run,
    single tokens handled by the decode kernel beside them."""
    dtype = torch.bfloat16
    cached = [5, 300, 0, 40, 0, 130, 700]
    new = [1, 1, 33, 70, 2, 129, 200]
    scale = 1.0 / math.sqrt(d)
    qkv, kp, vp, bt, step, ks, vs, cu = paged_case(cached, new, nh, nkv, d, ps, dtype, seed=nh + 3)
    want = reference_attention(qkv, ks, vs, cu, cached, new, nh, nkv, d, scale, window)
    for wide in (False, True):
        with attention_constants(PREFILL_WIDE_MIN_GROUPS=0 if wide else 1 << 30, **key_runs(splits)):
            got = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, window)
            torch.testing.assert_close(got.float().cpu(), want, **tol(dtype, 2e-5, 2e-2))
            whole = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, window, force="prefill")
            torch.testing.assert_close(whole.float().cpu(), want, **tol(dtype, 2e-5, 2e-2))


@pytest.mark.parametrize("kind,dtype", kinds_and_dtypes("generic", "prefill", "decode"))
@pytest.mark.parametrize("window", [1, 7, 64, 100])
def test_attention_window(ops, dtype, kind, window, decode_kind):
    nh, nkv, d, ps = 6, 2, 32, 8
    cached, new = ([0, 30, 200, 99], [50, 90, 3, 1]) if kind != "decode" else ([0, 30, 200, 99, 6], [1] * 5)
    scale = 0.2
    qkv, kp, vp, bt, step, ks, vs, cu = paged_case(cached, new, nh, nkv, d, ps, dtype, seed=window)
    got = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, window, force=kind)
    want = reference_attention(qkv, ks, vs, cu, cached, new, nh, nkv, d, scale, window)
    torch.testing.assert_close(got.float().cpu(), want, **tol(dtype, 2e-5, 2e-2))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,ps", LAYOUTS)
def test_attention_decode(ops, dtype, nh, nkv, d, ps, decode_kind):
    """One token per sequence, 37 context lengths 1 + (i * 53) % 700 as in the reference's
    kernel test (crates/model/src/paged_attention.rs:461-527), unsplit and split."""
    lens = [1 + (i * 53) % 700 for i in range(37)]
    cached, new = [l - 1 for l in lens], [1] * len(lens)
    scale = 1.0 / math.sqrt(d)
    qkv, kp, vp, bt, step, ks, vs, cu = paged_case(cached, new, nh, nkv, d, ps, dtype, seed=d)
    want = reference_attention(qkv, ks, vs, cu, cached, new, nh, nkv, d, scale, None)
    for part_keys, max_parts in DECODE_CUTS:
        with attention_constants(DECODE_PART_KEYS=part_keys, DECODE_MAX_PARTS=max_parts):
            got = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, None, force="decode")
        torch.testing.assert_close(got.float().cpu(), want, **tol(dtype, 2e-5, 2e-2))
    got = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, None)
    torch.testing.assert_close(got.float().cpu(), want, **tol(dtype, 2e-5, 2e-2))


@pytest.mark.parametrize("nh,nkv,d,ps,rotate", [(32, 8, 64, 16, True), (24, 8, 128, 16, True),
                                                (16, 2, 256, 16, True), (8, 8, 64, 32, False),
                                                (5, 5, 48, 16, True), (9, 3, 112, 16, False)])
@pytest.mark.parametrize("window", [None, 100])
def test_rope_attention_decode_in_one_kernel(ops, nh, nkv, d, ps, rotate, window):
    """The decode kernel that rotates q and k and stores the new k, v itself against
    rope_kv_write followed by attention: same output, same pages; with and without a cache
    write, unsplit and split (the new key then belongs to the last partition that has keys).
    Head sizes 48 and 112 with rotation take the two-kernel path inside rope_attention."""
    dtype = torch.bfloat16
    lens = [1 + (i * 53) % 700 for i in range(19)] + [256, 257, 512, 513, 1]
    cached, new = [l - 1 for l in lens], [1] * len(lens)
    scale = 1.0 / math.sqrt(d)
    qkv, kp, vp, bt, step, ks, vs, cu = paged_case(cached, new, nh, nkv, d, ps, dtype, seed=d + 1)
    cos = sin = None
    if rotate:
        ang = rnd(max(lens) + 1, d // 2, seed=5, scale=3.0)
        cos, sin = torch.cos(ang), torch.sin(ang)
    tables = bt.cpu()
    slots = torch.tensor([int(tables[s, (l - 1) // ps]) * ps + (l - 1) % ps for s, l in enumerate(lens)],
                         dtype=torch.int32, device=DEV)
    for write_kv in (True, False):
        for part_keys, max_parts in DECODE_CUTS:
            results = []
            for fused in (False, True):
                q2, k2, v2 = qkv.clone(), kp.clone(), vp.clone()
                old = ops.FUSE_ROPE_DECODE
                try:
                    ops.FUSE_ROPE_DECODE = fused
                    with attention_constants(DECODE_PART_KEYS=part_keys, DECODE_MAX_PARTS=max_parts):
                        out = ops.rope_attention(q2, nh, nkv, d, cos, sin, step.positions, slots, k2,
                                                 v2, ps, bt, step, scale, window, write_kv=write_kv)
                finally:
                    ops.FUSE_ROPE_DECODE = old
                results.append((out.float().cpu(), k2.float().cpu(), v2.cpu()))
            (o0, k0, v0), (o1, k1, v1) = results
            torch.testing.assert_close(o1, o0, atol=2e-2, rtol=2e-2)
            torch.testing.assert_close(k1, k0, atol=2e-2, rtol=1e-2)      # one rounding apart at most
            assert torch.equal(v1, v0)
            if not write_kv:
                assert torch.equal(k1, kp.float().cpu()) and torch.equal(v1, vp.cpu())


@pytest.mark.parametrize("nh,nkv,d,ps", [(32, 8, 64, 16), (24, 8, 128, 16), (8, 2, 256, 16), (8, 8, 64, 32),
                                         (5, 5, 48, 16), (34, 2, 64, 16), (16, 2, 256, 16)])
@pytest.mark.parametrize("window", [None, 70])
def test_rope_attention_turns_queries_inside_the_prefill_kernel(ops, nh, nkv, d, ps, window):
    """A batch with portions of prompts: rope_kv_write leaves q alone and the matrix-core
    kernels (prefill for the portions in tiles of 64 and of 128 queries and with their keys cut
    into runs, decode for the single tokens that lead the batch) turn each query as they load
    it, against rope_kv_write on all heads followed by attention: same output within a
    rounding, the very same pages, q left unrotated.  Head size 48, and groups of query heads
    that the decode kernel does not take (17 heads per KV head; 8 heads of 256 dims) with
    single tokens in the batch, take the two-kernel path inside rope_attention."""
    dtype = torch.bfloat16
    cached = [5, 63, 300, 0, 40, 0, 130, 17, 2100, 700]
    new = [1, 1, 1, 33, 70, 2, 129, 64, 150, 300]
    scale = 1.0 / math.sqrt(d)
    qkv, kp, vp, bt, step, ks, vs, cu = paged_case(cached, new, nh, nkv, d, ps, dtype, seed=d + 3)
    ang = rnd(max(c + n for c, n in zip(cached, new)) + 1, d // 2, seed=7, scale=3.0)
    cos, sin = torch.cos(ang), torch.sin(ang)
    tables = bt.cpu()
    slots = torch.tensor([int(tables[s, p // ps]) * ps + p % ps
                          for s, (c, n) in enumerate(zip(cached, new)) for p in range(c, c + n)],
                         dtype=torch.int32, device=DEV)
    results = []
    for fused in (False, True):
        q2, k2, v2 = qkv.clone(), kp.clone(), vp.clone()
        old = ops.FUSE_ROPE_PREFILL
        try:
            ops.FUSE_ROPE_PREFILL = fused
            out = ops.rope_attention(q2, nh, nkv, d, cos, sin, step.positions, slots, k2, v2, ps,
                                     bt, step, scale, window)
        finally:
            ops.FUSE_ROPE_PREFILL = old
        results.append((out.float().cpu(), q2.cpu(), k2.cpu(), v2.cpu()))
    (o0, q0, k0, v0), (o1, q1, k1, v1) = results
    torch.testing.assert_close(o1, o0, atol=2e-2, rtol=2e-2)
    assert torch.equal(k1, k0) and torch.equal(v1, v0)
    g = nh // nkv
    takes_it = d in (64, 128, 256) and g <= 16 and g * (d + 2) * 32 <= 65536
    assert torch.equal(q1[:, :nh * d], qkv.cpu()[:, :nh * d]) == takes_it
    assert not torch.equal(q0[:, :nh * d], qkv.cpu()[:, :nh * d])
    # and the rotated queries' result is the plain one over the keys that the pages now hold
    for s, (c, n) in enumerate(zip(cached, new)):
        for p in range(c, c + n):
            ks[s][p] = k0[int(tables[s, p // ps]), :, p % ps, :].float()
            vs[s][p] = v0[int(tables[s, p // ps]), :, :, p % ps].float()
    want = reference_attention(q0, ks, vs, cu, cached, new, nh, nkv, d, scale, window)
    torch.testing.assert_close(o1, want, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_decode_long_split(ops, dtype, decode_kind):
    """Long contexts beside short ones with many partitions, some of them empty
    (lens [1, 5, 300, 4000, 9000]: paged_attention.rs:503-527)."""
    nh, nkv, d, ps = 8, 2, 64, 16
    lens = [1, 5, 300, 4000, 9000]
    cached, new = [l - 1 for l in lens], [1] * len(lens)
    scale = 1.0 / math.sqrt(d)
    qkv, kp, vp, bt, step, ks, vs, cu = paged_case(cached, new, nh, nkv, d, ps, dtype, seed=9)
    want = reference_attention(qkv, ks, vs, cu, cached, new, nh, nkv, d, scale, None)
    for part_keys, max_parts in ((1024, 16), (256, 36), (256, 5)):
        with attention_constants(DECODE_PART_KEYS=part_keys, DECODE_MAX_PARTS=max_parts):
            got = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, None, force="decode")
        torch.testing.assert_close(got.float().cpu(), want, **tol(dtype, 2e-5, 2e-2))


@pytest.mark.parametrize("nh,nkv,d,ps", [(32, 8, 64, 16), (24, 8, 128, 16), (16, 2, 256, 16), (5, 5, 48, 16),
                                         (9, 3, 112, 16)])
@pytest.mark.parametrize("window", [None, 700])
def test_attention_decode_partitions_merged_inside_the_kernel(ops, nh, nkv, d, ps, window):
    """The matrix-core decode kernel merging a sequence's partitions itself (the last workgroup
    to finish does it) against the same kernel followed by the merge kernel: bit for bit the
    same, whichever workgroup comes last, and again on every further call (the arrival counts
    go back to zero by themselves).  Sequences with one partition beside ones with many, and a
    grid deeper than most sequences need.  The counts live in the caller's memory: a call with
    counters of its own gives the same floats and leaves them zero, and a second caller's
    counters are not touched by it."""
    dtype = torch.bfloat16
    lens = [1, 5, 300, 1024, 1025, 2100, 4000, 9000, 255, 256, 257, 3, 2048, 2049]
    cached, new = [l - 1 for l in lens], [1] * len(lens)
    scale = 1.0 / math.sqrt(d)
    qkv, kp, vp, bt, step, ks, vs, cu = paged_case(cached, new, nh, nkv, d, ps, dtype, seed=d + 3)
    want = reference_attention(qkv, ks, vs, cu, cached, new, nh, nkv, d, scale, window)
    old = ops.MERGE_DECODE_INSIDE, ops.MERGE_DECODE_INSIDE_MAX_BYTES
    try:
        ops.MERGE_DECODE_INSIDE_MAX_BYTES = 1 << 50          # whatever the size of the grid
        for part_keys, max_parts in ((1024, 16), (256, 36), (256, 5), (512, 2)):
            with attention_constants(DECODE_PART_KEYS=part_keys, DECODE_MAX_PARTS=max_parts):
                ops.MERGE_DECODE_INSIDE = False
                outside = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, window,
                                              force="decode")
                torch.testing.assert_close(outside.float().cpu(), want, **tol(dtype, 2e-5, 2e-2))
                ops.MERGE_DECODE_INSIDE = True
                for call in range(3):
                    inside = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale,
                                                 window, force="decode")
                    assert torch.equal(inside, outside), f"cut {part_keys} x {max_parts}, call {call}"
                mine = torch.zeros(len(lens) * nkv, dtype=torch.int32, device=DEV)
                other = torch.full((64,), 7, dtype=torch.int32, device=DEV)
                for call in range(2):
                    inside = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale,
                                                 window, force="decode", counters=mine)
                    assert torch.equal(inside, outside)
                    assert int(mine.abs().sum()) == 0 and int((other - 7).abs().sum()) == 0
                # fewer counters than (sequence, KV head) pairs: the second kernel merges
                few = torch.zeros(len(lens) * nkv - 1, dtype=torch.int32, device=DEV)
                inside = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, window,
                                             force="decode", counters=few)
                assert torch.equal(inside, outside) and int(few.abs().sum()) == 0
    finally:
        ops.MERGE_DECODE_INSIDE, ops.MERGE_DECODE_INSIDE_MAX_BYTES = old


@pytest.mark.parametrize("nh,nkv,d,ps,rotate", [(32, 8, 64, 16, True), (24, 8, 128, 16, True),
                                                (8, 2, 256, 16, True), (5, 5, 48, 16, False),
                                                (9, 3, 112, 16, False)])
@pytest.mark.parametrize("window", [None, 700])
def test_attention_decode_workgroups_that_walk_partitions(ops, nh, nkv, d, ps, rotate, window):
    """A workgroup of the matrix-core decode kernel that takes several partitions in a row
    (what a full batch gets instead of one workgroup per partition) against one workgroup per
    partition: the same floats for every walk, in the output and in the pages, since the
    partitions, their sums and the order of the merge stay what the sequence's own length makes
    them.  The kernel rotates and stores the step's own key itself here; the walking form waits
    for that store in front of its last round of chunks only.  Contexts end at, just before
    and just behind the edges of partitions and of rounds; a walk whose parked sums do not fit
    the LDS is refused."""
    from rust_llm_inference_server_amd.ops import attention_plan
    from rust_llm_inference_server_amd.ops.lib import KernelError
    dtype = torch.bfloat16
    lens = [1, 300, 512, 513, 1024, 1025, 1026, 1280, 1281, 1536, 1537, 2047, 2048, 2049, 2100,
            3000, 4000, 5000]
    cached, new = [l - 1 for l in lens], [1] * len(lens)
    scale = 1.0 / math.sqrt(d)
    qkv, kp, vp, bt, step, ks, vs, cu = paged_case(cached, new, nh, nkv, d, ps, dtype, seed=d + 7)
    cos = sin = None
    if rotate:
        ang = rnd(max(lens) + 1, d // 2, seed=6, scale=3.0)
        cos, sin = torch.cos(ang), torch.sin(ang)
    tables = bt.cpu()
    slots = torch.tensor([int(tables[s, (l - 1) // ps]) * ps + (l - 1) % ps for s, l in enumerate(lens)],
                         dtype=torch.int32, device=DEV)
    room = attention_plan.decode_walk_room(nh // nkv, d)
    old = ops.DECODE_WALK, ops.MERGE_DECODE_INSIDE_MAX_BYTES
    try:
        ops.MERGE_DECODE_INSIDE_MAX_BYTES = 1 << 50
        for part_keys, max_parts in ((1024, 16), (512, 16), (512, 2)):
            with attention_constants(DECODE_PART_KEYS=part_keys, DECODE_MAX_PARTS=max_parts):
                results = {}
                for walk in (1, 2, 3, 5, 16):
                    ops.DECODE_WALK = walk
                    q2, k2, v2 = qkv.clone(), kp.clone(), vp.clone()
                    deep = min(walk, attention_plan.decode_depth(max(lens)))   # what is asked for
                    if deep > 1 and deep > room:
                        with pytest.raises(KernelError, match="walks several partitions"):
                            ops.rope_attention(q2, nh, nkv, d, cos, sin, step.positions, slots, k2, v2,
                                               ps, bt, step, scale, window)
                        continue
                    out = ops.rope_attention(q2, nh, nkv, d, cos, sin, step.positions, slots, k2, v2,
                                             ps, bt, step, scale, window)
                    results[walk] = (out.cpu(), k2.cpu(), v2.cpu())
                o1, k1, v1 = results.pop(1)
                assert not torch.equal(k1, kp.cpu())                  # the new keys were stored
                for walk, (o, k, v) in results.items():
                    where = f"cut {part_keys} x {max_parts}, walk {walk}"
                    assert torch.equal(o, o1), where
                    assert torch.equal(k, k1) and torch.equal(v, v1), where
    finally:
        ops.DECODE_WALK, ops.MERGE_DECODE_INSIDE_MAX_BYTES = old


@pytest.mark.parametrize("kind,dtype", kinds_and_dtypes("generic", "prefill", "decode"))
def test_attention_finds_a_far_key(ops, dtype, kind, decode_kind):
    """One key among hundreds is made to stand out (its key vector equals the scaled query
    direction); the output must be that key's value, wherever its page lies."""
    nh, nkv, d, ps = 4, 2, 64, 16
    total = 777
    cached, new = ([total - 1], [1]) if kind == "decode" else ([total - 3], [3])
    qkv, kp, vp, bt, step, ks, vs, cu = paged_case(cached, new, nh, nkv, d, ps, dtype, seed=5)
    far = 131                                   # in the middle of a page, far from the end
    table = bt[0].tolist()
    qdir = qkv[-1, :d].float()                  # last token, head 0 (KV head 0)
    kp[table[far // ps], 0, far % ps, :] = (qdir * 50.0 / qdir.norm()).to(dtype)
    ks[0][far, 0, :] = kp[table[far // ps], 0, far % ps, :].float().cpu()
    scale = 1.0
    got = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, None, force=kind)
    want = reference_attention(qkv, ks, vs, cu, cached, new, nh, nkv, d, scale, None)
    torch.testing.assert_close(got.float().cpu(), want, **tol(dtype, 2e-5, 2e-2))
    torch.testing.assert_close(got[-1, :d].float().cpu(), vs[0][far, 0, :], **tol(dtype, 1e-4, 2e-2))


def alone(step, s, cached, new, bt, qkv, cu, ps):
    """The step, block table and queries of sequence ``s`` of a batch as a batch of its own (same
    pages)."""
    one = FakeStep()
    n, c = new[s], cached[s]
    one.num_tokens, one.num_seqs = n, 1
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    one.cu_seqlens, one.start_pos, one.ctx_lens = i32([0, n]), i32([c]), i32([c + n])
    one.positions, one.seq_of_token = i32(list(range(c, c + n))), i32([0] * n)
    one.max_context, one.max_new, one.all_decode = c + n, n, n == 1
    one.num_single = 1 if n == 1 else 0
    one.lengths = StepLengths(np.asarray([c], dtype=np.int64), np.asarray([n], dtype=np.int64),
                              one.num_single, ps)
    return one, bt[s:s + 1].contiguous(), qkv[cu[s]:cu[s + 1]].contiguous()


@pytest.mark.parametrize("nh,nkv,d,ps", [(32, 8, 64, 16), (24, 8, 128, 16), (6, 2, 32, 8)])
@pytest.mark.parametrize("window", [None, 700])
def test_attention_rows_do_not_depend_on_the_neighbours(ops, nh, nkv, d, ps, window):
    """bfloat16: the rows of a sequence come out bit for bit the same when it is alone in the
    step as among others, whatever they bring: decode partitions, tile form and key runs follow
    from its own lengths.  Long contexts beside short ones, portions that take key runs (few
    tiles on a long context) beside ones that do not, tiles of 128 queries beside tiles of 64."""
    dtype = torch.bfloat16
    scale = 1.0 / math.sqrt(d)
    # single tokens first, as the engine's steps order them; contexts on both sides of 1024,
    # 2048 and 4096 positions
    cached = [0, 1023, 1024, 2500, 4200, 0, 3000, 100, 2047, 4000]
    new = [1, 1, 1, 1, 1, 300, 200, 700, 70, 130]
    qkv, kp, vp, bt, step, ks, vs, cu = paged_case(cached, new, nh, nkv, d, ps, dtype, seed=d + 7)
    assert step.num_single == 5
    together = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, window)
    want = reference_attention(qkv, ks, vs, cu, cached, new, nh, nkv, d, scale, window)
    torch.testing.assert_close(together.float().cpu(), want, **tol(dtype, 2e-5, 2e-2))
    planner = ops.attention_planner(nh, nkv, d, dtype)
    forms = {planner.tile_queries(c, n) for c, n in zip(cached[5:], new[5:])}
    runs = {planner.key_runs(c, n, planner.tile_queries(c, n)) for c, n in zip(cached[5:], new[5:])}
    if d <= 128:
        assert forms == {64, 128}
    assert 1 in runs and max(runs) > 1                      # the batch mixes all of it
    for s in range(len(new)):
        one, table, q = alone(step, s, cached, new, bt, qkv, cu, ps)
        got = ops.paged_attention(q, nh, nkv, d, kp, vp, ps, table, one, scale, window)
        assert torch.equal(got, together[cu[s]:cu[s + 1]]), f"sequence {s}"
    # the single tokens as a decode step of their own, and in another order
    order = [3, 0, 4, 2, 1]
    sub = FakeStep()
    sub.num_tokens = sub.num_seqs = sub.num_single = 5
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    sub.cu_seqlens, sub.start_pos = i32(list(range(6))), i32([cached[s] for s in order])
    sub.ctx_lens = i32([cached[s] + 1 for s in order])
    sub.positions, sub.seq_of_token = sub.start_pos, i32(list(range(5)))
    sub.max_context, sub.max_new, sub.all_decode = max(cached[:5]) + 1, 1, True
    sub.lengths = StepLengths(np.asarray([cached[s] for s in order], dtype=np.int64),
                              np.ones(5, dtype=np.int64), 5, ps)
    got = ops.paged_attention(qkv[order].contiguous(), nh, nkv, d, kp, vp, ps,
                              bt[order].contiguous(), sub, scale, window)
    assert torch.equal(got, together[order])


@pytest.mark.parametrize("kind,dtype", kinds_and_dtypes("generic", "prefill", "decode"))
@pytest.mark.parametrize("window", [5, 64, 100, 300])
def test_attention_window_edge(ops, dtype, kind, window, decode_kind):
    """The last query sees keys p - window + 1 .. p.  The key just outside the window is made
    to stand out: it must not be seen.  Then the first key inside is made to stand out twice as
    much: the output must be its value.  An edge that is off by one fails one of the two."""
    nh, nkv, d, ps = 4, 2, 64, 16
    total = 555
    cached, new = ([total - 1], [1]) if kind == "decode" else ([total - 3], [3])
    qkv, kp, vp, bt, step, ks, vs, cu = paged_case(cached, new, nh, nkv, d, ps, dtype, seed=window)
    table = bt[0].tolist()
    qdir = qkv[-1, :d].float()                  # last token, head 0 (KV head 0)
    qdir = qdir / qdir.norm()
    p = total - 1

    def stand_out(pos, by):
        kp[table[pos // ps], 0, pos % ps, :] = (qdir * by).to(dtype)
        ks[0][pos, 0, :] = kp[table[pos // ps], 0, pos % ps, :].float().cpu()

    def run():
        got = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, 1.0, window, force=kind)
        want = reference_attention(qkv, ks, vs, cu, cached, new, nh, nkv, d, 1.0, window)
        torch.testing.assert_close(got.float().cpu(), want, **tol(dtype, 2e-5, 2e-2))
        return got[-1, :d].float().cpu()

    stand_out(p - window, 50.0)
    unseen = run()
    assert (unseen - vs[0][p - window, 0, :]).abs().max() > 0.1
    stand_out(p - window + 1, 100.0)
    seen = run()
    torch.testing.assert_close(seen, vs[0][p - window + 1, 0, :], **tol(dtype, 1e-4, 2e-2))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,ps", [(6, 2, 32, 8), (5, 5, 48, 16), (32, 8, 64, 16)])
def test_attention_with_a_bias_on_the_scores(ops, dtype, nh, nkv, d, ps):
    """slope[h] * (key position - query position) added to the scores before the softmax (a
    position encoding that works on the scores; the reference has none): portions beside single
    tokens and single tokens alone, with and without a window, through the kernels that the
    batch takes by itself (bfloat16: the matrix-core kernels' forms with a bias, over several
    decode partitions and key runs too; float32: the vector-unit kernels) and through the
    generic kernel, against the plain attention with the bias as an additive mask.  A slope so
    steep that only the query's own position counts returns that position's value."""
    scale = 1.0 / math.sqrt(d)
    slopes = torch.tensor([0.5 ** (1 + h % 5) for h in range(nh)], dtype=torch.float32)

    def reference(qkv, ks, vs, cu, cached, new, sl, window):
        outs = []
        q_all = qkv.float().cpu()[:, :nh * d]
        for s, (c, n) in enumerate(zip(cached, new)):
            q = q_all[cu[s]:cu[s + 1]].reshape(n, nh, d).transpose(0, 1)
            k, v = ks[s].transpose(0, 1), vs[s].transpose(0, 1)
            dist = torch.arange(c + n).reshape(1, -1) - torch.arange(c, c + n).reshape(-1, 1)
            mask = plain.causal_mask(n, c, window)
            o = torch.stack([plain.gqa_attention(q[h:h + 1], k[h // (nh // nkv):h // (nh // nkv) + 1],
                                                 v[h // (nh // nkv):h // (nh // nkv) + 1],
                                                 mask + sl[h] * dist, scale)[0] for h in range(nh)])
            outs.append(o.transpose(0, 1).reshape(n, nh * d))
        return torch.cat(outs)

    for cached, new in (([0, 5, 40, 130, 17], [33, 1, 70, 2, 64]), ([4, 99, 0, 640], [1, 1, 1, 1]),
                        ([1, 1100], [1, 1]), ([1200, 2], [1, 130])):
        for window in (None, 50):
            qkv, kp, vp, bt, step, ks, vs, cu = paged_case(cached, new, nh, nkv, d, ps, dtype, seed=nh + 9)
            want = reference(qkv, ks, vs, cu, cached, new, slopes, window)
            with attention_constants(DECODE_PART_KEYS=256, **key_runs(3)):
                for force in (None, "generic"):
                    got = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, window,
                                              bias_slopes=slopes.to(DEV), force=force)
                    torch.testing.assert_close(got.float().cpu(), want, **tol(dtype, 2e-5, 2e-2))
            plainly = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, window)
            assert (got.float() - plainly.float()).abs().max().item() > 1e-2       # the bias matters
    steep = torch.full((nh,), 1000.0, dtype=torch.float32, device=DEV)
    qkv, kp, vp, bt, step, ks, vs, cu = paged_case([30, 7], [1, 1], nh, nkv, d, ps, dtype, seed=3)
    got = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, None, bias_slopes=steep)
    for s, last in enumerate((30, 7)):
        for h in range(nh):
            torch.testing.assert_close(got[s, h * d:(h + 1) * d].float().cpu(), vs[s][last, h // (nh // nkv)],
                                       **tol(dtype, 1e-5, 1e-2))
    if dtype == torch.bfloat16:
        # tiles of 128 queries (two query blocks a wave) take the bias too
        qkv, kp, vp, bt, step, ks, vs, cu = paged_case([20], [300], nh, nkv, d, ps, dtype, seed=5)
        want = reference(qkv, ks, vs, cu, [20], [300], slopes, None)
        with attention_constants(PREFILL_WIDE_MIN_GROUPS=0):
            got = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, scale, None,
                                      bias_slopes=slopes.to(DEV), force="prefill")
        torch.testing.assert_close(got.float().cpu(), want, **tol(dtype, 2e-5, 2e-2))


@pytest.mark.parametrize("dtype", DTYPES)
def test_rope_interleaved_layout(ops, dtype):
    """The rotation that pairs dim 2j with 2j + 1 (the reference rotates halves): against the
    formula, over part of the head, into the pages; position 0 is the identity."""
    T, nh, nkv, d, rot, ps = 9, 3, 1, 48, 32, 8
    inv = plain.inv_freqs(rot, 10000.0, None)
    positions = torch.tensor([0, 1, 5, 63, 17, 2, 3, 40, 8], dtype=torch.int32)
    cos, sin = plain.rope_tables(inv, positions.tolist())
    cos_all, sin_all = plain.rope_tables(inv, range(64))
    qkv = rnd(T, (nh + 2 * nkv) * d, dtype=dtype, seed=12)
    src = qkv.float().cpu()
    slots = torch.arange(T, dtype=torch.int32) + 3
    kp = torch.zeros(4, nkv, ps, d, dtype=dtype, device=DEV)
    vp = torch.zeros(4, nkv, d, ps, dtype=dtype, device=DEV)
    ops.rope_kv_write(qkv, nh, nkv, d, cos_all.to(DEV), sin_all.to(DEV), positions.to(DEV), slots.to(DEV),
                      kp, vp, ps, interleaved=True)

    def rotated(x):                                  # x (T, heads, d)
        out = x.clone()
        a, b = x[..., 0:rot:2], x[..., 1:rot:2]
        c, s = cos.unsqueeze(1), sin.unsqueeze(1)
        out[..., 0:rot:2] = a * c - b * s
        out[..., 1:rot:2] = b * c + a * s
        return out

    want_q = rotated(src[:, :nh * d].reshape(T, nh, d)).reshape(T, nh * d)
    torch.testing.assert_close(qkv[:, :nh * d].float().cpu(), want_q, **tol(dtype, 1e-5, 2e-2))
    want_k = rotated(src[:, nh * d:(nh + nkv) * d].reshape(T, nkv, d))
    for t in range(T):
        slot = int(slots[t])
        torch.testing.assert_close(kp[slot // ps, :, slot % ps, :].float().cpu(), want_k[t],
                                   **tol(dtype, 1e-5, 2e-2))
    assert torch.equal(qkv[0, :nh * d].float().cpu(), src[0, :nh * d])         # position 0
    # not the rotation of halves
    halves = qkv.clone()
    halves[:] = rnd(T, (nh + 2 * nkv) * d, dtype=dtype, seed=12)
    ops.rope_kv_write(halves, nh, nkv, d, cos_all.to(DEV), sin_all.to(DEV), positions.to(DEV), None, None,
                      None, ps, write_kv=False)
    assert (halves[1:, :nh * d].float() - qkv[1:, :nh * d].float()).abs().max().item() > 0.1


def test_attention_one_key_returns_its_value(ops):
    nh, nkv, d, ps = 4, 2, 32, 8
    for kind in ("generic", "decode"):
        qkv, kp, vp, bt, step, ks, vs, cu = paged_case([0, 0], [1, 1], nh, nkv, d, ps, torch.float32)
        got = ops.paged_attention(qkv, nh, nkv, d, kp, vp, ps, bt, step, 0.3, None, force=kind)
        for s in range(2):
            for h in range(nh):
                torch.testing.assert_close(got[s, h * d:(h + 1) * d].cpu(), vs[s][0, h // 2],
                                           atol=1e-6, rtol=1e-6)


# ------------------------------------------------------------------------ sampling
def test_sample_rows_greedy_and_ties(ops):
    # the reference's vector: ties go to the lowest index (crates/model/src/sampling.rs:184-199)
    logits = torch.tensor([[0.1, 3.0, -1.0, 3.0], [5.0, 1.0, 5.0, 0.0]], device=DEV)
    zeros_i = torch.zeros(2, dtype=torch.int32, device=DEV)
    zeros_f = torch.zeros(2, device=DEV)
    assert ops.sample_rows(logits, zeros_i, zeros_f).tolist() == [1, 0]
    neg = torch.tensor([[float("-inf"), -5.0]], device=DEV)
    assert ops.sample_rows(neg, zeros_i[:1], zeros_f[:1]).tolist() == [1]
    big = rnd(5, 128256, seed=3)
    got = ops.sample_rows(big, torch.zeros(5, dtype=torch.int32, device=DEV), torch.zeros(5, device=DEV))
    assert got.tolist() == big.argmax(dim=-1).tolist()
    # a vocabulary scanned in chunks: equal maxima in different chunks, and a row of -inf
    wide = torch.full((3, 70001), -1.0, device=DEV)
    wide[0, 69999] = wide[0, 1234] = wide[0, 40000] = 2.0
    wide[1, 70000] = 0.5
    wide[2] = float("-inf")
    zi, zf = torch.zeros(3, dtype=torch.int32, device=DEV), torch.zeros(3, device=DEV)
    assert ops.sample_rows(wide, zi, zf).tolist() == [1234, 70000, 0]


def test_sample_rows_temperature_matches_host_reference(ops):
    V = 50021
    logits = rnd(6, V, seed=11) * 2
    keys = [plain.row_key(42 + r, 100 + r) for r in range(6)]
    inv_t = [1 / 0.7, 1 / 0.8, 0.0, 1 / 1.3, 1 / 0.1, 1.0]
    kt = torch.tensor([k - (1 << 32) if k >= (1 << 31) else k for k in keys], dtype=torch.int32, device=DEV)
    got = ops.sample_rows(logits, kt, torch.tensor(inv_t, device=DEV)).tolist()
    want = [plain.sample_row(logits[r].cpu(), keys[r], inv_t[r]) for r in range(6)]
    assert got == want
    # the same key gives the same token whatever the neighbours are
    again = ops.sample_rows(logits[3:4].contiguous(), kt[3:4].contiguous(),
                            torch.tensor(inv_t[3:4], device=DEV)).tolist()
    assert again == got[3:4]


def test_sample_rows_frequencies_follow_softmax(ops):
    # crates/model/src/sampling.rs:216-241: l = [0, 1, 2, -1], T = 0.7, 20,000 keys, within 0.015
    n = 20000
    l = torch.tensor([0.0, 1.0, 2.0, -1.0])
    logits = l.repeat(n, 1).to(DEV)
    keys = [plain.row_key(42, i) for i in range(n)]
    kt = torch.tensor([k - (1 << 32) if k >= (1 << 31) else k for k in keys], dtype=torch.int32, device=DEV)
    got = ops.sample_rows(logits, kt, torch.full((n,), 1 / 0.7, device=DEV))
    freq = torch.bincount(got.long().cpu(), minlength=4).float() / n
    want = torch.softmax(l / 0.7, dim=0)
    assert (freq - want).abs().max().item() < 0.015


# ---------------------------------------------------------------------- page copies
@pytest.mark.parametrize("dtype", DTYPES)
def test_copy_pages(ops, dtype):
    pages = rnd(3, 10, 2, 8, 16, dtype=dtype)
    src = torch.tensor([1, 7], dtype=torch.int32, device=DEV)
    dst = torch.tensor([4, 0], dtype=torch.int32, device=DEV)
    want = pages.clone()
    want[:, 4], want[:, 0] = pages[:, 1], pages[:, 7]
    ops.copy_pages(pages, src, dst)
    torch.testing.assert_close(pages, want, atol=0, rtol=0)


# ------------------------------------------------------------------ large pools
@pytest.mark.parametrize("dtype", DTYPES)
def test_pages_past_two_to_the_31_elements(ops, dtype):
    """A pool whose last pages start beyond element 2^31 of the K and V arrays (a few GB per
    layer, small on a 288 GB card): cache write, the three attention kernels and the page copy
    give bit for bit what they give for the same pages at the start of a small pool."""
    nh, nkv, d, ps = 8, 8, 64, 16
    cached, new = [0, 40, 130, 17, 300], [33, 2, 70, 1, 1]
    scale = 1.0 / math.sqrt(d)
    qkv, kp, vp, bt, step, ks, vs, cu = paged_case(cached, new, nh, nkv, d, ps, dtype, seed=2)
    small = kp.shape[0]
    big = (1 << 31) // (nkv * ps * d) + small + 5
    shift = big - small
    kb = torch.empty(big, nkv, ps, d, dtype=dtype, device=DEV)
    vb = torch.empty(big, nkv, d, ps, dtype=dtype, device=DEV)
    assert kb[shift:].storage_offset() > (1 << 31)
    kb[shift:], vb[shift:] = kp, vp
    bt_big = bt + shift
    inv = plain.inv_freqs(d, 10000.0, None)
    cos, sin = (t.to(DEV) for t in plain.rope_tables(inv, range(512)))
    tables = bt.cpu()
    pos = step.positions.cpu().tolist()
    seq = step.seq_of_token.cpu().tolist()
    slots = torch.tensor([int(tables[s, p // ps]) * ps + p % ps for s, p in zip(seq, pos)],
                         dtype=torch.int32, device=DEV)
    q_small, q_big = qkv.clone(), qkv.clone()
    ops.rope_kv_write(q_small, nh, nkv, d, cos, sin, step.positions, slots, kp, vp, ps)
    ops.rope_kv_write(q_big, nh, nkv, d, cos, sin, step.positions, slots + shift * ps, kb, vb, ps)
    assert torch.equal(q_small, q_big)
    assert torch.equal(kb[shift:], kp) and torch.equal(vb[shift:], vp)
    kinds = ["generic"] + (["prefill"] if dtype == torch.bfloat16 else [])
    for kind in kinds:
        a = ops.paged_attention(q_small, nh, nkv, d, kp, vp, ps, bt, step, scale, None, force=kind)
        b = ops.paged_attention(q_big, nh, nkv, d, kb, vb, ps, bt_big, step, scale, None, force=kind)
        assert torch.equal(a, b), kind
    # single tokens: the decode kernels, with and without the rotation and cache write inside
    lens = [c + n for c, n in zip(cached, new)]
    dq, _, _, _, dstep, *_ = paged_case([l - 1 for l in lens], [1] * len(lens), nh, nkv, d, ps, dtype, seed=3)
    with attention_constants(DECODE_PART_KEYS=256):
        a = ops.paged_attention(dq, nh, nkv, d, kp, vp, ps, bt, dstep, scale, None, force="decode")
        b = ops.paged_attention(dq, nh, nkv, d, kb, vb, ps, bt_big, dstep, scale, None, force="decode")
    assert torch.equal(a, b)
    dslots = torch.tensor([int(tables[s, (l - 1) // ps]) * ps + (l - 1) % ps for s, l in enumerate(lens)],
                          dtype=torch.int32, device=DEV)
    a = ops.rope_attention(dq.clone(), nh, nkv, d, cos, sin, dstep.positions, dslots, kp, vp, ps, bt,
                           dstep, scale, None)
    b = ops.rope_attention(dq.clone(), nh, nkv, d, cos, sin, dstep.positions, dslots + shift * ps, kb, vb,
                           ps, bt_big, dstep, scale, None)
    assert torch.equal(a, b)
    assert torch.equal(kb[shift:], kp) and torch.equal(vb[shift:], vp)
    # page copy to and from the far end
    pool = kb.reshape(1, big, -1)
    src = torch.tensor([shift + 1, 0], dtype=torch.int32, device=DEV)
    dst = torch.tensor([2, big - 1], dtype=torch.int32, device=DEV)
    first, far = pool[0, 0].clone(), pool[0, shift + 1].clone()
    ops.copy_pages(pool, src, dst)
    assert torch.equal(pool[0, 2], far) and torch.equal(pool[0, big - 1], first)


def test_seeded_weights_made_on_the_device_are_the_hosts(ops):
    """The seeded generator on the device against the host's (one formula, twice written): the
    float32 values agree to the bit but for a library's last digit of log and cos in double
    precision (one float32 step, next to never); bfloat16 is the float32 value rounded."""
    from rust_llm_inference_server_amd.weights.random_init import normal_fill
    for n, seed, tensor, mean, std in ((1, 0, 0, 0.0, 0.02), (7, 5, 3, 1.0, 0.02),
                                       (300001, 2 ** 63 + 9, 146, 0.0, 0.02)):
        want = normal_fill(n, seed, tensor, mean, std)
        got = torch.empty(n, dtype=torch.float32, device=DEV)
        ops.fill_normal(got, seed, tensor, mean, std)
        got = got.cpu()
        step = torch.maximum(want.abs(), torch.tensor(1e-30)) * 2.0 ** -23
        assert ((got - want).abs() <= step).all()
        assert (got != want).sum().item() <= max(1, n // 100000)
        half = torch.empty(n, dtype=torch.bfloat16, device=DEV)
        ops.fill_normal(half, seed, tensor, mean, std)
        assert (half.cpu() != got.to(torch.bfloat16)).sum().item() == 0


# ----------------------------------------------------------------- refusals
def test_kernels_refuse_what_they_cannot_do(ops):
    with pytest.raises(ops.KernelError):
        ops.linear(rnd(2, 8), rnd(3, 9))
    with pytest.raises(ops.KernelError):
        ops.swiglu(rnd(2, 7))
    with pytest.raises(ops.KernelError):
        ops.embed(torch.zeros(2, dtype=torch.int32), torch.zeros(4, 4))       # CPU tensors
    qkv, kp, vp, bt, step, *_ = paged_case([0], [4], 2, 1, 24, 8, torch.bfloat16)
    with pytest.raises(ops.KernelError):           # head_dim 24 is no multiple of 16
        ops.paged_attention(qkv, 2, 1, 24, kp, vp, 8, bt, step, 1.0, None, force="prefill")
