"""Each kernel alone against its plain reference, at sizes other than the tiny engines': widths
and vocabularies that are no power of two, several head sizes and group sizes, scrambled
pages, windows, long contexts with one far key made to stand out."""

from __future__ import annotations

import math
import random

import pytest
import torch

from plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from turboserve_amd.kernels.ops import Ops

    return Ops(DEV)


def tol(dtype):
    return dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


# -- rows -------------------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("tokens,hidden", [(1, 72), (5, 3584), (3, 1100), (2, 4100)])
def test_rmsnorm_and_fused_residual(ops, dtype, tokens, hidden):
    g = torch.Generator().manual_seed(hidden)
    x = (torch.randn(tokens, hidden, generator=g) * 3).to(dtype)
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(dtype)
    eps = 1e-5
    want = plain.rms_norm(x.float(), w.float(), eps)
    got = ops.rmsnorm(x.to(DEV), w.to(DEV), eps).float().cpu()
    torch.testing.assert_close(got, want, **tol(dtype))

    residual = torch.randn(tokens, hidden, generator=g)
    total = residual + x.float()
    res_dev = residual.to(DEV)
    got = ops.add_rmsnorm(res_dev, x.to(DEV), w.to(DEV), eps).float().cpu()
    torch.testing.assert_close(res_dev.cpu(), total, rtol=0, atol=1e-6)  # the sum is kept in 32-bit
    torch.testing.assert_close(got, plain.rms_norm(total, w.float(), eps), **tol(dtype))

    rows = torch.tensor([tokens - 1, 0], dtype=torch.int32, device=DEV)
    res_dev = residual.to(DEV)
    got = ops.add_rmsnorm(res_dev, x.to(DEV), w.to(DEV), eps, rows).float().cpu()
    torch.testing.assert_close(res_dev.cpu(), residual, rtol=0, atol=0)  # untouched with rows
    torch.testing.assert_close(got, plain.rms_norm(total, w.float(), eps)[[tokens - 1, 0]], **tol(dtype))


def test_rmsnorm_rounds_before_the_gain(ops):
    """bfloat16: the normalised value is rounded to bfloat16 before the gain multiplies it
    (src/turboserve/engine/model/layers.py:208); a single rounding of the product differs."""
    g = torch.Generator().manual_seed(3)
    x = torch.randn(64, 512, generator=g).bfloat16()
    w = (1 + 0.3 * torch.randn(512, generator=g)).bfloat16()
    want = plain.rms_norm(x, w, 1e-6)  # bfloat16 in, reference order of roundings
    got = ops.rmsnorm(x.to(DEV), w.to(DEV), 1e-6).cpu()
    assert (got != want).float().mean() < 0.01  # rsqrt may differ in the last bit now and then
    single = (w.float() * (x.float() * torch.rsqrt((x.float() ** 2).mean(-1, keepdim=True) + 1e-6))).bfloat16()
    assert (single != want).float().mean() > 0.02


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed_swiglu_gather(ops, dtype):
    g = torch.Generator().manual_seed(0)
    table = torch.randn(301, 72, generator=g).to(dtype)
    ids = torch.tensor([5, 300, 0, 5], dtype=torch.int32)
    got = ops.embed(table.to(DEV), ids.to(DEV)).cpu()
    assert got.dtype == torch.float32
    torch.testing.assert_close(got, table.float()[ids.long()], rtol=0, atol=0)

    gu = torch.randn(7, 2 * 200, generator=g).to(dtype)
    want = torch.nn.functional.silu(gu.float()[:, :200]) * gu.float()[:, 200:]
    torch.testing.assert_close(ops.swiglu(gu.to(DEV)).float().cpu(), want, **tol(dtype))
    zero_up = gu.clone()
    zero_up[:, 200:] = 0
    assert float(ops.swiglu(zero_up.to(DEV)).abs().max()) == 0.0
    # the same values with gate and up alternating, for widths that take the 8-wide kernel (bfloat16), the
    # 4-wide one and neither, over more rows than a workgroup has threads
    for rows, inter in ((7, 200), (7, 201), (7, 204), (300, 72)):
        gu = torch.randn(rows, 2 * inter, generator=g).to(dtype)
        want = torch.nn.functional.silu(gu.float()[:, :inter]) * gu.float()[:, inter:]
        pairs = torch.stack([gu[:, :inter], gu[:, inter:]], dim=2).reshape(rows, 2 * inter).contiguous()
        halves = ops.swiglu(gu.to(DEV)).cpu()
        torch.testing.assert_close(halves.float(), want, **tol(dtype))
        assert torch.equal(ops.swiglu(pairs.to(DEV), paired=True).cpu(), halves)

    rows = torch.tensor([6, 0, 3], dtype=torch.int32)
    torch.testing.assert_close(ops.gather_rows(gu.to(DEV), rows.to(DEV)).cpu(), gu[rows.long()], rtol=0, atol=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [(1, 7, 5), (3, 130, 100), (16, 50, 64), (32, 33, 130), (33, 17, 65), (70, 65, 33), (130, 320, 96),
                                   (97, 129, 17), (300, 257, 200)])
def test_gemm_plain(ops, dtype, m, n, k):
    g = torch.Generator().manual_seed(m * n)
    x = torch.randn(m, k, generator=g).to(dtype)
    w = torch.randn(n, k, generator=g).to(dtype)
    b = torch.randn(n, generator=g).to(dtype)
    want = x.double() @ w.double().T + b.double()
    got = ops.gemm_plain(x.to(DEV), w.to(DEV), b.to(DEV)).double().cpu()
    bound = 1e-5 if dtype == torch.float32 else 2e-2
    assert float((got - want).abs().max()) <= bound * math.sqrt(k) * 4
    got32 = ops.gemm_plain(x.to(DEV), w.to(DEV), out_float32=True)
    assert got32.dtype == torch.float32
    assert float((got32.double().cpu() - x.double() @ w.double().T).abs().max()) <= 1e-5 * math.sqrt(k) * 4
    zero = ops.gemm_plain(x.to(DEV), torch.zeros_like(w).to(DEV), b.to(DEV)).float().cpu()
    torch.testing.assert_close(zero, b.float().expand(m, n), rtol=0, atol=0)  # a dropped bias would show


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("k", [200, 64, 131, 1])
def test_gemm_plain_rows_do_not_depend_on_the_batch(ops, dtype, k):
    """The same bits for a row whatever the batch: alone, among a few rows (the layout for up to
    32 rows, one output a thread), among many (tiles of 64 x 64): every output is the same chain
    of fused multiply-adds in the order of k in both layouts."""
    g = torch.Generator().manual_seed(9)
    x = torch.randn(300, k, generator=g).to(dtype)
    w = torch.randn(150, k, generator=g).to(dtype)
    b = torch.randn(150, generator=g).to(dtype)
    full = ops.gemm_plain(x.to(DEV), w.to(DEV), b.to(DEV)).cpu()
    for rows in (slice(40, 41), slice(0, 8), slice(20, 45), slice(3, 35), slice(10, 43), slice(0, 64), slice(100, 196),
                 slice(7, 104), slice(150, 300)):
        part = ops.gemm_plain(x[rows].to(DEV), w.to(DEV), b.to(DEV)).cpu()
        assert torch.equal(full[rows], part), rows


@pytest.mark.parametrize("m", [1, 5, 16, 17, 33, 64, 65, 100, 128])
@pytest.mark.parametrize("n,k", [(7, 8), (130, 104), (320, 96), (3584, 1000), (301, 2056), (4608, 3584), (33000, 136)])
def test_gemm_skinny(ops, m, n, k):
    """The decode-sized product: 32-bit partial sums over ranges of K whose sum is the product,
    for row counts around the 16-row tiles, N that is no multiple of a tile or of 4, K that is
    no multiple of the kernels' depth (128 and 256), one split and many, a matrix wide enough
    for the resident kernel to take the fewest rows."""
    g = torch.Generator().manual_seed(m * n + k)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.1).bfloat16()
    b = torch.randn(n, generator=g).bfloat16()
    want = x.double() @ w.double().T + b.double()
    bound = 2e-5 * math.sqrt(k) * float(want.abs().max() + 1)
    products = [lambda **kw: ops.gemm_skinny(x.to(DEV), w.to(DEV), b.to(DEV), **kw),
                lambda **kw: ops.gemm_tiled(x.to(DEV), w.to(DEV), b.to(DEV), **kw)]
    if m <= 16:
        products.append(lambda **kw: ops.gemm_resident(x.to(DEV), w.to(DEV), b.to(DEV), **kw))
    for product in products:
        for max_splits in (None, 1):
            partial = product(max_splits=max_splits)
            assert partial.dtype == torch.float32 and partial.shape[1:] == (m, n)
            if max_splits == 1:
                assert partial.shape[0] == 1
            assert float((partial.double().sum(0).cpu() - want).abs().max()) <= bound
    none = ops.gemm_skinny(x.to(DEV), torch.zeros_like(w).to(DEV), b.to(DEV)).sum(0).cpu()
    torch.testing.assert_close(none, b.float().expand(m, n), rtol=0, atol=0)  # the bias, once


@pytest.mark.parametrize("tile", [2, 4, 5, 8])
@pytest.mark.parametrize("m,n,k", [(64, 500, 1096), (3, 161, 128), (16, 200, 392), (17, 333, 264), (32, 96, 1096), (40, 64, 40),
                                   (128, 330, 520), (77, 1000, 264)])
def test_gemm_tiled_every_tile_and_grid(ops, tile, m, n, k):
    """The tiled product with its grid given by hand: every tile size, ranges of K of one
    iteration and of several, a last range that is shorter, a last tile of rows that is partly
    beyond N, a K below one iteration.  Tiles of 256 weight rows take up to 32 rows and refuse
    more."""
    if tile == 8 and m > 32:
        x = torch.zeros(m, k).bfloat16().to(DEV)
        with pytest.raises(Exception, match="ts_gemm_tiled"):
            ops.gemm_tiled(x, torch.zeros(n, k).bfloat16().to(DEV), plan=(-(-k // 128), 1, tile))
        return
    g = torch.Generator().manual_seed(tile * 1000 + n)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.1).bfloat16()
    want = x.double() @ w.double().T
    iters = -(-k // 128)
    for per_split in sorted({1, 2, iters, max(1, iters - 1)}):
        splits = -(-iters // per_split)
        partial = ops.gemm_tiled(x.to(DEV), w.to(DEV), plan=(per_split, splits, tile))
        assert partial.shape == (splits, m, n)
        got = partial.double().sum(0).cpu()
        assert float((got - want).abs().max()) <= 2e-5 * math.sqrt(k) * float(want.abs().max() + 1), per_split


@pytest.mark.parametrize("tile,m,inter,k", [(t, *c) for t in (2, 4, 5, 8) for c in (
    (64, 250, 264), (5, 81, 128), (16, 81, 392), (24, 250, 264), (33, 1000, 40), (128, 250, 264), (90, 81, 128)) if t != 8 or c[0] <= 32])
def test_gemm_tiled_applies_swiglu_itself(ops, tile, m, inter, k):
    """A gate|up matrix with alternating rows through the tiled product with the activation in
    its epilogue gives, bit for bit, what the product's partial sums followed by the SwiGLU
    kernel give; and the plain value of silu(x Wg^T) * (x Wu^T).  `linear_swiglu` takes that
    path when the product is one range of K, the two-kernel path otherwise, 32-bit included."""
    g = torch.Generator().manual_seed(tile + inter)
    x = torch.randn(m, k, generator=g).bfloat16()
    gate = (torch.randn(inter, k, generator=g) * 0.2).bfloat16()
    up = (torch.randn(inter, k, generator=g) * 0.2).bfloat16()
    w = torch.stack([gate, up], dim=1).reshape(2 * inter, k).contiguous()
    plan = (-(-k // 128), 1, tile)
    fused = ops.gemm_tiled(x.to(DEV), w.to(DEV), plan=plan, gated=True)
    two_steps = ops.swiglu(ops.gemm_tiled(x.to(DEV), w.to(DEV), plan=plan), torch.bfloat16, paired=True)
    assert fused.shape == (m, inter) and torch.equal(fused, two_steps)
    want = torch.nn.functional.silu(x.double() @ gate.double().T) * (x.double() @ up.double().T)
    assert float((fused.double().cpu() - want).abs().max()) <= 1e-2 * float(want.abs().max() + 1)
    either = ops.linear_swiglu(x.to(DEV), w.to(DEV))
    assert float((either.double().cpu() - want).abs().max()) <= 1e-2 * float(want.abs().max() + 1)
    exact = ops.linear_swiglu(x.float().to(DEV), w.float().to(DEV))
    assert exact.dtype == torch.float32
    assert float((exact.double().cpu() - want).abs().max()) <= 1e-5 * float(want.abs().max() + 1) * math.sqrt(k)
    with pytest.raises(Exception, match="one range of K"):
        ops.gemm_tiled(x.to(DEV), w.to(DEV), plan=(1, -(-k // 128), tile), gated=True) if k > 128 else ops.gemm_tiled(
            x.to(DEV), w.to(DEV), torch.zeros(2 * inter).bfloat16().to(DEV), plan=plan, gated=True)


WIDE_GRIDS = [(2, 128, 4), (4, 128, 4), (5, 128, 4), (2, 256, 4), (4, 256, 4), (5, 256, 4),
              (2, 128, 8), (4, 128, 8), (5, 128, 8), (2, 256, 8), (4, 256, 8), (5, 256, 8), (8, 256, 8)]


@pytest.mark.parametrize("tile,x_rows,waves", WIDE_GRIDS)
@pytest.mark.parametrize("m,n,k", [(130, 97, 72), (300, 500, 200), (257, 322, 136), (513, 640, 1096), (129, 1000, 40)])
def test_gemm_wide_every_tile_and_grid(ops, tile, x_rows, waves, m, n, k):
    """The product for steps of many rows with its grid given by hand: every tile of weight rows,
    both heights of the activation tile, four and eight wavefronts, one range of K (a bfloat16
    result with the bias) and several (32-bit partial sums), last tiles partly beyond N and M, a K
    that is no multiple of the 64 an iteration takes and one below it; and the SwiGLU in the
    product's epilogue against the two-kernel way."""
    g = torch.Generator().manual_seed(tile * 1000 + n + x_rows + waves)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.1).bfloat16()
    b = torch.randn(n, generator=g).bfloat16()
    want = x.double() @ w.double().T + b.double()
    iters = -(-k // 64)
    one = ops.gemm_wide(x.to(DEV), w.to(DEV), b.to(DEV), plan=(iters, 1, tile, x_rows, waves))
    assert one.shape == (m, n) and one.dtype == torch.bfloat16
    assert float((one.double().cpu() - want).abs().max()) <= 1e-2 * float(want.abs().max() + 1)
    for per_split in sorted({1, 2, max(1, iters - 1)}):
        splits = -(-iters // per_split)
        if splits == 1:
            continue
        partial = ops.gemm_wide(x.to(DEV), w.to(DEV), b.to(DEV), plan=(per_split, splits, tile, x_rows, waves))
        assert partial.shape == (splits, m, n) and partial.dtype == torch.float32
        got = partial.double().sum(0).cpu()
        assert float((got - want).abs().max()) <= 2e-5 * math.sqrt(k) * float(want.abs().max() + 1), per_split
    if n % 2 == 0:
        fused = ops.gemm_wide(x.to(DEV), w.to(DEV), plan=(iters, 1, tile, x_rows, waves), gated=True)
        two_steps = ops.swiglu(ops.gemm_wide(x.to(DEV), w.to(DEV), plan=(iters, 1, tile, x_rows, waves)), paired=True)
        y = x.double() @ w.double().T
        gated = torch.nn.functional.silu(y[:, 0::2]) * y[:, 1::2]
        assert fused.shape == (m, n // 2)
        assert float((fused.double().cpu() - gated).abs().max()) <= 1e-2 * float(gated.abs().max() + 1)
        # the fused form rounds once, the two-kernel form twice: equal up to that
        assert float((fused.double() - two_steps.double()).abs().max()) <= 1e-2 * float(gated.abs().max() + 1)
    with pytest.raises(Exception, match="one range of K"):
        ops.gemm_wide(x.to(DEV), w.to(DEV), plan=(1, iters, tile, x_rows, waves), gated=True) if iters > 1 else ops.gemm_wide(
            x.to(DEV), w.to(DEV), b.to(DEV), plan=(iters, 1, tile, x_rows, waves), gated=True)


@pytest.mark.parametrize("tile,x_rows,depth", [(2, 64, 64), (4, 64, 64), (5, 64, 64), (8, 64, 64), (2, 64, 128), (4, 64, 128),
                                                (5, 64, 128), (8, 128, 64)])
@pytest.mark.parametrize("m,n,k", [(40, 97, 72), (64, 500, 200), (33, 322, 1096), (17, 1000, 40), (100, 161, 264)])
def test_gemm_wide_at_decode_sizes(ops, tile, x_rows, depth, m, n, k):
    """The same kernel as the product of decode steps of 17 to 128 rows: tiles of 64 activation
    rows, iterations 64 and 128 deep, always partial sums out (or the SwiGLU), against the exact
    product; and `gemm_skinny` / `linear_swiglu`, which pick it for these row counts."""
    if m > x_rows:
        pytest.skip("one tile of activation rows here")
    g = torch.Generator().manual_seed(tile * 100 + n + depth)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.1).bfloat16()
    b = torch.randn(n, generator=g).bfloat16()
    want = x.double() @ w.double().T + b.double()
    iters = -(-k // depth)
    for per_split in sorted({1, iters}):
        splits = -(-iters // per_split)
        partial = ops.gemm_wide(x.to(DEV), w.to(DEV), b.to(DEV), plan=(per_split, splits, tile, x_rows, 8, depth), sums=True)
        assert partial.shape == (splits, m, n) and partial.dtype == torch.float32
        assert float((partial.double().sum(0).cpu() - want).abs().max()) <= 2e-5 * math.sqrt(k) * float(want.abs().max() + 1)
    picked = ops.gemm_skinny(x.to(DEV), w.to(DEV), b.to(DEV))
    assert float((picked.double().sum(0).cpu() - want).abs().max()) <= 2e-5 * math.sqrt(k) * float(want.abs().max() + 1)
    if n % 2 == 0:
        y = x.double() @ w.double().T
        gated = torch.nn.functional.silu(y[:, 0::2]) * y[:, 1::2]
        fused = ops.gemm_wide(x.to(DEV), w.to(DEV), plan=(iters, 1, tile, x_rows, 8, depth), gated=True)
        assert float((fused.double().cpu() - gated).abs().max()) <= 1e-2 * float(gated.abs().max() + 1)
        either = ops.linear_swiglu(x.to(DEV), w.to(DEV))
        assert float((either.double().cpu() - gated).abs().max()) <= 1e-2 * float(gated.abs().max() + 1)


def test_gemm_wide_rows_do_not_depend_on_the_batch_and_plans_fill_the_device(ops):
    """A row's result is the same bits whatever rows stand beside it (for one grid), rows behind
    the step's own reach nothing, and the planner's grids for the 7B shape's matrices give most
    compute units a workgroup."""
    g = torch.Generator().manual_seed(77)
    x = torch.randn(300, 264, generator=g).bfloat16().to(DEV)
    w = (torch.randn(500, 264, generator=g) * 0.1).bfloat16().to(DEV)
    plan = (5, 1, 4, 128, 8)
    whole = ops.gemm_wide(x, w, plan=plan)
    assert torch.equal(ops.gemm_wide(x[100:260], w, plan=plan), whole[100:260])
    shuffled = torch.randperm(300, generator=g).to(DEV)
    assert torch.equal(ops.gemm_wide(x[shuffled], w, plan=plan), whole[shuffled])
    for n, k in ((4608, 3584), (3584, 3584), (37888, 3584), (3584, 18944)):
        for m in (130, 256, 512, 1000):
            for one_range in (False, True):
                per_split, splits, tile, x_rows, waves = ops._wide_plan(m, n, k, one_range)
                assert splits == -(-(-(-k // 64)) // per_split) and (splits == 1 or not one_range)
                workgroups = -(-n // (32 * tile)) * -(-m // x_rows) * splits
                assert one_range or workgroups >= 0.8 * ops.compute_units, (m, n, k, workgroups)
    # through `linear`: 200 rows take the own kernel by default, and give the library's result up to rounding
    y = ops.linear(x[:200], w)
    assert y.dtype == torch.bfloat16 and y.shape == (200, 500)
    torch.testing.assert_close(y.float(), x[:200].float() @ w.float().t(), rtol=2e-2, atol=2e-2)
    sums = ops.linear(x[:200], w, for_residual=True)
    torch.testing.assert_close(ops.dense(sums, torch.bfloat16).float(), x[:200].float() @ w.float().t(), rtol=2e-2, atol=2e-2)


def test_library_product_at_a_larger_size_ignores_the_rows_behind(ops, monkeypatch):
    """With sizes set for the library's products, a step's activations are allocated up to the
    next size and the product runs that long; the rows behind the step's own (not-a-numbers
    here) reach no row of the result, and a buffer without the room runs at its own size.
    (The engine's own product for such steps is switched off here.)"""
    from turboserve_amd.kernels.ops import Ops

    monkeypatch.setattr(Ops, "wide_default_rows", 0)
    sized = Ops(DEV)
    sized.library_buckets = (192, 256)
    g = torch.Generator().manual_seed(12)
    x = torch.randn(150, 264, generator=g).bfloat16()
    w = (torch.randn(136, 264, generator=g) / 16).bfloat16()
    b = torch.randn(136, generator=g).bfloat16()
    ref = x.float() @ w.float().t()
    buffer = sized.rows_buffer(150, 264, torch.bfloat16, DEV)
    assert buffer.shape == (150, 264) and buffer.untyped_storage().nbytes() == 192 * 264 * 2
    buffer.as_strided((192, 264), (264, 1)).fill_(float("nan"))
    buffer.copy_(x)
    lengths = []
    mm, addmm = torch.mm, torch.addmm
    try:
        torch.mm = lambda a, *rest, **kw: (lengths.append(a.shape[0]), mm(a, *rest, **kw))[1]
        torch.addmm = lambda c, a, *rest, **kw: (lengths.append(a.shape[0]), addmm(c, a, *rest, **kw))[1]
        got = sized.linear(buffer, w.to(DEV))
        biased = sized.linear(buffer, w.to(DEV), b.to(DEV))
        wide = sized.linear_float32_out(buffer, w.to(DEV))
        tight = sized.linear(x.to(DEV), w.to(DEV))
        unsized = ops.linear(buffer, w.to(DEV))
    finally:
        torch.mm, torch.addmm = mm, addmm
    assert lengths == [192, 192, 192, 150, 150]
    for result in (got, tight, unsized):
        assert result.shape == (150, 136)
        torch.testing.assert_close(result.float().cpu(), ref, rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(biased.float().cpu(), ref + b.float(), rtol=2e-2, atol=3e-2)
    assert wide.dtype == torch.float32 and wide.shape == (150, 136)
    torch.testing.assert_close(wide.cpu(), ref, rtol=2e-2, atol=2e-2)


def test_gemm_skinny_rows_do_not_depend_on_the_batch(ops):
    """A row's sums are the same bits whatever else is in the batch, for a given grid of the
    tiled kernel and within the resident kernel; between grids the ranges of K differ, so only
    the rounding of 32-bit sums does."""
    g = torch.Generator().manual_seed(4)
    x = torch.randn(40, 1000, generator=g).bfloat16()
    w = torch.randn(200, 1000, generator=g).bfloat16()
    plan = (3, 3, 2)
    full = ops.gemm_tiled(x.to(DEV), w.to(DEV), plan=plan).cpu()
    some = ops.gemm_tiled(x[10:30].to(DEV), w.to(DEV), plan=plan).cpu()
    one = ops.gemm_tiled(x[17:18].to(DEV), w.to(DEV), plan=plan).cpu()
    assert torch.equal(full[:, 17:18], some[:, 7:8]) and torch.equal(full[:, 17:18], one)
    small = ops.gemm_resident(x[5:21].to(DEV), w.to(DEV)).cpu()
    nine = ops.gemm_resident(x[12:21].to(DEV), w.to(DEV)).cpu()
    alone = ops.gemm_resident(x[17:18].to(DEV), w.to(DEV)).cpu()
    assert torch.equal(small[:, 12:13], alone) and torch.equal(nine[:, 5:6], alone)
    torch.testing.assert_close(full.sum(0)[17:18], alone.sum(0), rtol=1e-5, atol=1e-3)
    other = ops.gemm_skinny(x.to(DEV), w.to(DEV)).cpu()  # the grid the engine would choose
    torch.testing.assert_close(full.sum(0), other.sum(0), rtol=1e-5, atol=1e-3)


@pytest.mark.parametrize("splits", [2, 3, 5, 8, 9, 16, 17, 29])
@pytest.mark.parametrize("hidden", [200, 201])
def test_consumers_add_up_partial_sums(ops, splits, hidden):
    """Norm, SwiGLU and rotary/cache write take the skinny product's 32-bit partial sums and
    give what they give for the summed tensor.  The kernels fetch the splits in batches (of 4,
    8, 16, and 8 at a time beyond that) and add them in split order: the residual they leave is,
    bit for bit, the residual plus the splits added one after the other.  Widths that are and
    are not a multiple of 4 take the kernels with and without 16-byte accesses."""
    from turboserve_amd.parts.rope import rotary_tables

    g = torch.Generator().manual_seed(8 + splits)
    tokens = 6
    parts = torch.randn(splits, tokens, hidden, generator=g)
    total = parts.sum(0)
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).bfloat16()
    residual = torch.randn(tokens, hidden, generator=g)
    res_dev = residual.to(DEV)
    got = ops.add_rmsnorm(res_dev, parts.to(DEV), w.to(DEV), 1e-6).float().cpu()
    in_order = residual.clone()
    for part in parts:
        in_order += part
    assert torch.equal(res_dev.cpu(), in_order)
    torch.testing.assert_close(got, plain.rms_norm(residual + total, w.float(), 1e-6), **tol(torch.bfloat16))
    rows = torch.tensor([4, 1], dtype=torch.int32, device=DEV)
    got = ops.add_rmsnorm(residual.to(DEV), parts.to(DEV), w.to(DEV), 1e-6, rows).float().cpu()
    torch.testing.assert_close(got, plain.rms_norm(residual + total, w.float(), 1e-6)[[4, 1]], **tol(torch.bfloat16))

    inter = 72 if hidden % 4 == 0 else 73
    gu = torch.randn(splits, tokens, 2 * inter, generator=g)
    want = torch.nn.functional.silu(gu.sum(0)[:, :inter]) * gu.sum(0)[:, inter:]
    torch.testing.assert_close(ops.swiglu(gu.to(DEV), torch.bfloat16).float().cpu(), want, **tol(torch.bfloat16))
    want = torch.nn.functional.silu(gu.sum(0)[:, 0::2]) * gu.sum(0)[:, 1::2]
    torch.testing.assert_close(ops.swiglu(gu.to(DEV), torch.bfloat16, paired=True).float().cpu(), want, **tol(torch.bfloat16))

    heads, kv_heads, dim, page = 3, 1, 32, 8
    proj = torch.randn(splits, tokens, (heads + 2 * kv_heads) * dim, generator=g)
    positions = torch.tensor([0, 5, 6, 30, 31, 2], dtype=torch.int32)
    slots = [3, 17, 9, 0, 25, 31]
    cos, sin = rotary_tables(64, dim, 1e4, 1.0)
    kp = torch.zeros(4, kv_heads, page, dim, dtype=torch.bfloat16, device=DEV)
    vp = torch.zeros(4, kv_heads, dim, page, dtype=torch.bfloat16, device=DEV)
    q, q_stride = ops.rope_store(proj.to(DEV), kp, vp, cos.to(DEV), sin.to(DEV), positions.to(DEV),
                                 torch.tensor(slots, dtype=torch.int32, device=DEV), heads, kv_heads, dim, page, 31,
                                 torch.bfloat16)
    assert q.shape == (tokens, heads * dim) and q_stride == heads * dim and q.dtype == torch.bfloat16
    summed = proj.sum(0)
    angles = plain.rope_angles(positions, dim, 1e4)
    q_want = plain.apply_rope(summed[:, : heads * dim].view(tokens, heads, dim), angles)
    k_want = plain.apply_rope(summed[:, heads * dim:(heads + kv_heads) * dim].view(tokens, kv_heads, dim), angles)
    v = summed[:, (heads + kv_heads) * dim:].view(tokens, kv_heads, dim)
    torch.testing.assert_close(q.float().cpu().view(tokens, heads, dim), q_want, **tol(torch.bfloat16))
    kp_want, vp_want = scatter_reference(k_want, v, slots, 4, kv_heads, page, dim)
    torch.testing.assert_close(kp.float().cpu(), kp_want, **tol(torch.bfloat16))
    torch.testing.assert_close(vp.float().cpu(), vp_want, **tol(torch.bfloat16))


# -- rotary + cache write ---------------------------------------------------------------------------


def scatter_reference(k, v, slots, num_pages, kv_heads, page, dim):
    """Key pages [NB, Hkv, BS, D] and transposed value pages [NB, Hkv, D, BS] after writing."""
    kp = torch.zeros(num_pages, kv_heads, page, dim)
    vp = torch.zeros(num_pages, kv_heads, dim, page)
    for t, slot in enumerate(slots):
        if slot < 0:
            continue
        kp[slot // page, :, slot % page, :] = k[t]
        vp[slot // page, :, :, slot % page] = v[t]
    return kp, vp


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dim,page,theta,factor", [(4, 2, 16, 16, 1e4, 1.0), (3, 1, 32, 8, 1e6, 1.0),
                                                                  (5, 5, 48, 32, 5e5, 2.0), (14, 2, 128, 16, 1e6, 1.0)])
def test_rope_store(ops, dtype, heads, kv_heads, dim, page, theta, factor):
    from turboserve_amd.parts.rope import rotary_tables

    g = torch.Generator().manual_seed(dim)
    tokens, num_pages = 9, 6
    qkv = torch.randn(tokens, (heads + 2 * kv_heads) * dim, generator=g).to(dtype)
    positions = torch.tensor([0, 1, 2, 40, 41, 7, 100, 3, 64], dtype=torch.int32)
    slot_pool = list(range(num_pages * page))
    random.Random(1).shuffle(slot_pool)
    slots = slot_pool[:tokens]
    slots[4] = -1  # no write for this token
    cos, sin = rotary_tables(128, dim, theta, factor)
    kp = torch.zeros(num_pages, kv_heads, page, dim, dtype=dtype, device=DEV)
    vp = torch.zeros(num_pages, kv_heads, dim, page, dtype=dtype, device=DEV)
    dev = qkv.to(DEV)
    ops.rope_store(dev, kp, vp, cos.to(DEV), sin.to(DEV), positions.to(DEV), torch.tensor(slots, dtype=torch.int32, device=DEV),
                   heads, kv_heads, dim, page, 100)
    q = qkv.float()[:, : heads * dim].view(tokens, heads, dim)
    k = qkv.float()[:, heads * dim:(heads + kv_heads) * dim].view(tokens, kv_heads, dim)
    v = qkv.float()[:, (heads + kv_heads) * dim:].view(tokens, kv_heads, dim)
    angles = plain.rope_angles(positions, dim, theta, factor)
    q_want, k_want = plain.apply_rope(q, angles), plain.apply_rope(k, angles)
    got = dev.float().cpu()
    torch.testing.assert_close(got[:, : heads * dim].view(tokens, heads, dim), q_want, **tol(dtype))
    # Only the queries are rotated in place; keys and values leave through the pages.
    torch.testing.assert_close(got[:, heads * dim:], qkv.float()[:, heads * dim:], rtol=0, atol=0)
    kp_want, vp_want = scatter_reference(k_want, v, slots, num_pages, kv_heads, page, dim)
    torch.testing.assert_close(kp.float().cpu(), kp_want, **tol(dtype))
    torch.testing.assert_close(vp.float().cpu(), vp_want, rtol=0, atol=0)
    with pytest.raises(Exception, match="beyond the rotary tables"):
        ops.rope_store(dev, kp, vp, cos.to(DEV), sin.to(DEV), positions.to(DEV), None, heads, kv_heads, dim, page, 128)


@pytest.mark.parametrize("heads,kv_heads,dim,page", [(7, 1, 128, 16), (3, 3, 48, 8), (4, 2, 32, 4), (2, 1, 96, 32)])
def test_rope_store_of_many_tokens_equals_token_by_token(ops, heads, kv_heads, dim, page):
    """Prompt portions of 32 tokens or more go through a kernel that handles 8 tokens per block
    with 16-byte accesses (values of 8 consecutive slots leave as one store into the transposed
    page).  It must write, bit for bit, what the per-token kernel writes when the same tokens
    come in pieces of fewer than 32: slots in runs that start on and off a multiple of 8, runs
    that cross pages, scattered slots, a token without a slot, a ragged last group."""
    from turboserve_amd.parts.rope import rotary_tables

    g = torch.Generator().manual_seed(dim + page)
    tokens, num_pages = 75, 256 // page + 1
    width = (heads + 2 * kv_heads) * dim
    qkv = torch.randn(tokens, width, generator=g).to(torch.bfloat16)
    positions = torch.cat([torch.arange(5, 45), torch.arange(0, 35)]).to(torch.int32)
    slots = list(range(16, 56))            # a run from a multiple of 8, over page edges
    slots += list(range(83, 83 + 19))      # a run that starts off a multiple of 8
    scattered = [3, 150, 7, 201, 130, 9, 64, 249, 11, 70, 2, 255, 128, 140, 0, 77]
    slots += scattered[: tokens - len(slots)]
    slots[50] = -1
    assert len(slots) == tokens and max(slots) < num_pages * page
    live = [s for s in slots if s >= 0]
    assert len(set(live)) == len(live)
    cos, sin = rotary_tables(64, dim, 10000.0, 1.0)
    cos, sin = cos.to(DEV), sin.to(DEV)
    results = []
    for piece in (tokens, 16):
        kp = torch.zeros(num_pages, kv_heads, page, dim, dtype=torch.bfloat16, device=DEV)
        vp = torch.zeros(num_pages, kv_heads, dim, page, dtype=torch.bfloat16, device=DEV)
        dev = qkv.to(DEV)
        for start in range(0, tokens, piece):
            stop = min(tokens, start + piece)
            ops.rope_store(dev[start:stop], kp, vp, cos, sin, positions[start:stop].to(DEV),
                           torch.tensor(slots[start:stop], dtype=torch.int32, device=DEV), heads, kv_heads, dim, page, 63)
        results.append((dev.cpu(), kp.cpu(), vp.cpu()))
    for whole, pieces in zip(*results):
        assert torch.equal(whole.view(torch.int16), pieces.view(torch.int16))
    # and against the plain rotation, so that both are not wrong together
    q = qkv.float()[:, : heads * dim].view(tokens, heads, dim)
    want = plain.apply_rope(q, plain.rope_angles(positions, dim, 10000.0, 1.0))
    torch.testing.assert_close(results[0][0].float()[:, : heads * dim].view(tokens, heads, dim), want, **tol(torch.bfloat16))


# -- attention --------------------------------------------------------------------------------------


class PagedCase:
    """Requests with dense random keys/values scattered into scrambled pages, and the plain
    attention of each request's last ``q_len`` positions."""

    def __init__(self, dtype, heads, kv_heads, dim, page, seqs, window=None, seed=0, spike=None):
        g = torch.Generator().manual_seed(seed)
        self.heads, self.kv_heads, self.dim, self.page, self.window = heads, kv_heads, dim, page, window
        self.seqs = seqs  # list of (context_len, query_len)
        need = sum(-(-c // page) for c, _ in seqs)
        num_pages = need + 3
        order = list(range(num_pages))
        random.Random(seed).shuffle(order)  # scrambled, interleaved block ids
        width = max(-(-c // page) for c, _ in seqs)
        self.table = torch.full((len(seqs), width), -1, dtype=torch.int32)
        self.kp = torch.randn(num_pages, kv_heads, page, dim, generator=g).to(dtype)  # stale data everywhere
        self.vp = torch.randn(num_pages, kv_heads, dim, page, generator=g).to(dtype)
        self.q, self.expected, self.positions, self.token_seq, self.qsl = [], [], [], [], [0]
        used = 0
        for s, (ctx, qlen) in enumerate(seqs):
            k = torch.randn(ctx, kv_heads, dim, generator=g).to(dtype)
            v = torch.randn(ctx, kv_heads, dim, generator=g).to(dtype)
            q = torch.randn(qlen, heads, dim, generator=g).to(dtype)
            if spike is not None and ctx > spike:
                # One far key dominates every query's scores: a kernel that skips it fails.
                k[spike] = 0
                k[spike, :, 0] = 16.0
                q[:] = 0
                q[:, :, 0] = 16.0
                v[spike] = 5.0
            pages = order[used:used + -(-ctx // page)]
            used += len(pages)
            self.table[s, : len(pages)] = torch.tensor(pages, dtype=torch.int32)
            for pos in range(ctx):
                self.kp[pages[pos // page], :, pos % page, :] = k[pos]
                self.vp[pages[pos // page], :, :, pos % page] = v[pos]
            qpos = torch.arange(ctx - qlen, ctx)
            mask = plain.attention_mask(qpos, ctx, window)
            self.expected.append(plain.attention(q.float(), k.float(), v.float(), mask, dim ** -0.5))
            self.q.append(q)
            self.positions.extend(qpos.tolist())
            self.token_seq.extend([s] * qlen)
            self.qsl.append(self.qsl[-1] + qlen)
        self.q = torch.cat(self.q).reshape(-1, heads * dim)
        self.expected = torch.cat(self.expected).reshape(-1, heads * dim)

    def dev(self, t, dtype=None):
        return (t if dtype is None else t.to(dtype)).to(DEV)

    def ints(self, values):
        return torch.tensor(values, dtype=torch.int32, device=DEV)


ATTENTION_GEOMETRIES = [
    # heads, kv_heads, dim, page
    (4, 2, 16, 16),
    (3, 1, 32, 8),
    (5, 5, 48, 32),
    (14, 2, 128, 16),   # G = 7, as the 7B shape
    (8, 1, 64, 16),
    (40, 2, 80, 16),    # G = 20: more than one tile of heads per KV head
    (2, 1, 256, 64),
    (6, 2, 256, 16),    # G = 3 at the largest head size: staged windows above 64 KiB of LDS
    (10, 2, 48, 8),     # G = 5, a head size that is no multiple of 32
    (9, 3, 32, 16),     # G = 3 at the smallest head size of the 32-tokens-per-wavefront prefill kernel
    (10, 2, 96, 32),    # G = 5 (two chunks of four heads, the second with one live wavefront), head size 96
    (40, 8, 128, 16),   # G = 5 on 8 KV heads, as the 14B and 32B shapes
    (14, 2, 64, 8),     # G = 7 on pages of 8 keys: the prefill kernel's wavefronts fetch for themselves
    (28, 2, 64, 32),    # G = 14: two workgroups of seven heads and a feeding wavefront per KV head
    (16, 1, 32, 16),    # G = 16: three workgroups of six heads, the last with four live ones
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dim,page", ATTENTION_GEOMETRIES)
@pytest.mark.parametrize("window", [None, 20])
def test_attention_generic(ops, dtype, heads, kv_heads, dim, page, window):
    case = PagedCase(dtype, heads, kv_heads, dim, page, [(70, 1), (33, 33), (90, 7), (1, 1), (129, 2)], window, seed=dim)
    got = ops.paged_attention_generic(
        case.dev(case.q), heads * dim, case.dev(case.kp), case.dev(case.vp), case.dev(case.table),
        case.ints(case.token_seq), case.ints(case.positions), heads, dim ** -0.5, window,
    ).float().cpu()
    torch.testing.assert_close(got, case.expected, **tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [None, 20])
def test_attention_generic_with_a_bias_by_distance(ops, dtype, window):
    """slopes[h] * (key - query position) is added to the scores before the softmax: with a steep
    slope a head attends to its own position only, with slope 0 it is plain attention, and in
    between it matches the formula written out."""
    heads, kv_heads, dim, page = 6, 2, 32, 8
    seqs = [(70, 5), (33, 33), (129, 2)]
    case = PagedCase(dtype, heads, kv_heads, dim, page, seqs, window, seed=3)
    slopes = torch.tensor([0.0, 0.03, 0.5, 1e4, 0.1, 2.0])
    got = ops.paged_attention_generic(
        case.dev(case.q), heads * dim, case.dev(case.kp), case.dev(case.vp), case.dev(case.table),
        case.ints(case.token_seq), case.ints(case.positions), heads, dim ** -0.5, window, slopes.to(DEV),
    ).float().cpu().view(-1, heads, dim)
    want = torch.empty_like(got)
    row = 0
    for s, (ctx, qlen) in enumerate(seqs):
        pages = case.table[s, : -(-ctx // page)].long()
        k = case.kp[pages].permute(0, 2, 1, 3).reshape(-1, kv_heads, dim)[:ctx].float()  # [ctx, Hkv, D]
        v = case.vp[pages].permute(0, 3, 1, 2).reshape(-1, kv_heads, dim)[:ctx].float()
        q = case.q[row:row + qlen].view(qlen, heads, dim).float()
        qpos = torch.arange(ctx - qlen, ctx)
        mask = plain.attention_mask(qpos, ctx, window)
        distance = (torch.arange(ctx)[None, :] - qpos[:, None]).float()
        for h in range(heads):
            scores = (q[:, h] @ k[:, h // 3].T) * dim ** -0.5 + slopes[h] * distance
            want[row:row + qlen, h] = torch.softmax(scores.masked_fill(~mask, float("-inf")), dim=-1) @ v[:, h // 3]
            if h == 3:  # the steep head sees its own key only
                torch.testing.assert_close(want[row:row + qlen, h], v[qpos, h // 3], rtol=0, atol=1e-6)
        row += qlen
    torch.testing.assert_close(got, want, **tol(dtype))
    torch.testing.assert_close(got[:, 0].reshape(-1), case.expected.view(-1, heads, dim)[:, 0].reshape(-1), **tol(dtype))


@pytest.mark.parametrize("heads,kv_heads,dim,page", ATTENTION_GEOMETRIES)
@pytest.mark.parametrize("window", [None, 20, 300])
def test_attention_decode_mfma(ops, heads, kv_heads, dim, page, window):
    contexts = [70, 1, 33, 600, 129, 32, 31, 257]
    case = PagedCase(torch.bfloat16, heads, kv_heads, dim, page, [(c, 1) for c in contexts], window, seed=dim + 1)
    out = torch.zeros(len(contexts), heads * dim, dtype=torch.bfloat16, device=DEV)
    ops.attention_decode(
        out, case.dev(case.q), heads * dim, case.dev(case.kp), case.dev(case.vp), case.dev(case.table),
        case.ints(case.qsl), case.ints(contexts), 0, len(contexts), heads, dim ** -0.5, window, max(contexts),
    )
    torch.testing.assert_close(out.float().cpu(), case.expected, **tol(torch.bfloat16))


def prefill_blocks_of(ops, case, heads, kv_heads, dim, seqs, shuffle=None):
    """(rows per block the kernel for this geometry takes, its work list for ``seqs``)."""
    rows = ops.prefill_block_rows(dim, heads, kv_heads)
    blocks = [(s, case.qsl[s] + off) for s, (_, qlen) in enumerate(seqs) for off in range(0, qlen, rows)]
    if shuffle is not None:
        random.Random(shuffle).shuffle(blocks)
    return rows, blocks


def test_attention_decode_mfma_far_key_and_subrange(ops):
    """A context of thousands of keys where one far key carries the result, split over many
    wavefronts; and a launch over a sub-range of the step's requests (rows before it untouched)."""
    heads, kv_heads, dim, page = 28, 4, 128, 16
    contexts = [4100, 3000, 5, 2049]
    case = PagedCase(torch.bfloat16, heads, kv_heads, dim, page, [(c, 1) for c in contexts], None, seed=5, spike=1234)
    out = torch.full((len(contexts), heads * dim), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.attention_decode(
        out, case.dev(case.q), heads * dim, case.dev(case.kp), case.dev(case.vp), case.dev(case.table),
        case.ints(case.qsl), case.ints(contexts), 1, 3, heads, dim ** -0.5, None, max(contexts),
    )
    got = out.float().cpu()
    assert float((got[0] - 7.0).abs().max()) == 0.0
    torch.testing.assert_close(got[1:], case.expected[1:], **tol(torch.bfloat16))
    assert float(case.expected[1].abs().mean()) > 4.0  # the spike's value dominates


def test_attention_decode_mfma_at_tens_of_thousands_of_keys(ops):
    """One request with 40,000 keys (the most splits a launch makes) next to a short one; a far
    key carries the long one's result."""
    heads, kv_heads, dim, page = 14, 2, 128, 16
    contexts = [40000, 700]
    case = PagedCase(torch.bfloat16, heads, kv_heads, dim, page, [(c, 1) for c in contexts], None, seed=9, spike=23456)
    out = torch.zeros(len(contexts), heads * dim, dtype=torch.bfloat16, device=DEV)
    ops.attention_decode(
        out, case.dev(case.q), heads * dim, case.dev(case.kp), case.dev(case.vp), case.dev(case.table),
        case.ints(case.qsl), case.ints(contexts), 0, len(contexts), heads, dim ** -0.5, None, max(contexts),
    )
    torch.testing.assert_close(out.float().cpu(), case.expected, **tol(torch.bfloat16))
    assert float(case.expected[0].abs().mean()) > 4.0
    # the same cache, its last 40 positions as a prompt portion
    seqs = [(40000, 40)]
    portion = PagedCase(torch.bfloat16, heads, kv_heads, dim, page, seqs, None, seed=9, spike=23456)
    rows, blocks = prefill_blocks_of(ops, portion, heads, kv_heads, dim, seqs)
    out = torch.zeros(40, heads * dim, dtype=torch.bfloat16, device=DEV)
    ops.attention_prefill(
        out, portion.dev(portion.q), heads * dim, portion.dev(portion.kp), portion.dev(portion.vp),
        portion.dev(portion.table), portion.ints(portion.qsl), portion.ints([40000]), portion.ints(blocks), heads,
        dim ** -0.5, None, 40000, rows,
    )
    torch.testing.assert_close(out.float().cpu(), portion.expected, **tol(torch.bfloat16))


@pytest.mark.parametrize("heads,kv_heads,dim,page", ATTENTION_GEOMETRIES)
@pytest.mark.parametrize("window", [None, 20, 300])
def test_attention_prefill_mfma(ops, heads, kv_heads, dim, page, window):
    """Whole prompts, portions that continue a cached prefix, two-token portions; block edges at
    every alignment against pages and 32-key windows."""
    seqs = [(70, 70), (33, 2), (600, 77), (129, 16), (257, 17), (48, 48), (2, 2), (515, 33)]
    case = PagedCase(torch.bfloat16, heads, kv_heads, dim, page, seqs, window, seed=dim + 2)
    rows, blocks = prefill_blocks_of(ops, case, heads, kv_heads, dim, seqs, shuffle=3)
    out = torch.zeros(case.qsl[-1], heads * dim, dtype=torch.bfloat16, device=DEV)
    ops.attention_prefill(
        out, case.dev(case.q), heads * dim, case.dev(case.kp), case.dev(case.vp), case.dev(case.table),
        case.ints(case.qsl), case.ints([c for c, _ in seqs]), case.ints(blocks), heads, dim ** -0.5, window,
        max(c for c, _ in seqs), rows,
    )
    torch.testing.assert_close(out.float().cpu(), case.expected, **tol(torch.bfloat16))


def test_prefill_block_rows_follow_the_geometry(ops):
    """32 rows per wavefront where the wide kernel runs (three or more query heads per KV head,
    head sizes 32 to 128 in steps of 32), 16 elsewhere; a work list of the other length is refused."""
    from turboserve_amd.kernels.ops import KernelError

    assert ops.prefill_block_rows(128, 28, 4) == 32 and ops.prefill_block_rows(64, 8, 1) == 32
    assert ops.prefill_block_rows(128, 8, 4) == 16 and ops.prefill_block_rows(48, 10, 2) == 16
    assert ops.prefill_block_rows(256, 6, 2) == 16 and ops.prefill_block_rows(80, 40, 2) == 16
    case = PagedCase(torch.bfloat16, 14, 2, 128, 16, [(40, 40)], None, seed=1)
    out = torch.zeros(40, 14 * 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(KernelError, match="rows"):
        ops.attention_prefill(out, case.dev(case.q), 14 * 128, case.dev(case.kp), case.dev(case.vp), case.dev(case.table),
                              case.ints(case.qsl), case.ints([40]), case.ints([(0, 0), (0, 16), (0, 32)]), 14, 128 ** -0.5,
                              None, 40, 16)


@pytest.mark.parametrize("heads,kv_heads,dim,tokens", [(14, 2, 128, 1200), (14, 2, 128, 3100), (14, 2, 64, 4200)])
def test_attention_prefill_mfma_every_launch_plan(ops, heads, kv_heads, dim, tokens):
    """The 32-tokens-per-wavefront kernel picks its form by the size of the grid (on 256 compute
    units: 1,200 tokens, fed workgroups on part of the device; 3,100 tokens, self-fed workgroups
    with heavy and light blocks paired; 4,200 tokens, more fed workgroups than compute units).
    One prompt each, beside a short portion at the end of another request."""
    seqs = [(tokens, tokens), (900, 70)]
    case = PagedCase(torch.bfloat16, heads, kv_heads, dim, 16, seqs, None, seed=tokens)
    rows, blocks = prefill_blocks_of(ops, case, heads, kv_heads, dim, seqs)
    assert rows == 32
    out = torch.zeros(case.qsl[-1], heads * dim, dtype=torch.bfloat16, device=DEV)
    ops.attention_prefill(
        out, case.dev(case.q), heads * dim, case.dev(case.kp), case.dev(case.vp), case.dev(case.table),
        case.ints(case.qsl), case.ints([c for c, _ in seqs]), case.ints(blocks), heads, dim ** -0.5, None, tokens, rows,
    )
    torch.testing.assert_close(out.float().cpu(), case.expected, **tol(torch.bfloat16))


def shared_out_work(case, seqs, window, shares_wanted):
    """A work list in which every block of 32 rows with two or more windows of keys is shared out
    over up to ``shares_wanted`` workgroups, written out from the entry point's description."""
    from turboserve_amd.kernels.ops import PrefillWork, prefill_block_windows

    blocks, ranges, combine, slot = [], [], [], 0
    for s, (ctx, qlen) in enumerate(seqs):
        for offset in range(0, qlen, 32):
            here = min(32, qlen - offset)
            windows = prefill_block_windows(ctx - qlen + offset, here, window or 0)
            shares = min(shares_wanted, windows)
            if shares < 2:
                blocks.append((s, case.qsl[s] + offset))
                ranges.append((0, 0, -1))
                continue
            each = -(-windows // shares)
            shares = -(-windows // each)
            combine.append((case.qsl[s] + offset, here, slot, shares))
            for share in range(shares):
                blocks.append((s, case.qsl[s] + offset))
                ranges.append((share * each, min(each, windows - share * each), slot))
                slot += 1
    order = list(range(len(blocks)))
    random.Random(5).shuffle(order)
    return PrefillWork(case.ints([blocks[i] for i in order]), case.ints([ranges[i] for i in order]),
                       case.ints(combine), slot)


@pytest.mark.parametrize("heads,kv_heads,dim,page", [g for g in ATTENTION_GEOMETRIES if g[0] // g[1] >= 3 and g[2] % 32 == 0 and g[2] <= 128])
@pytest.mark.parametrize("window", [None, 20, 300])
@pytest.mark.parametrize("shares", [2, 3, 16])
def test_attention_prefill_mfma_with_shared_out_blocks(ops, heads, kv_heads, dim, page, window, shares):
    """The keys of a block shared out over two, three and sixteen workgroups (fewer where a block
    has fewer windows; a share of one window included), whole blocks beside them, ragged last
    blocks, windows that cut shares off from some rows: the combined result is the plain one."""
    seqs = [(70, 70), (33, 2), (600, 77), (129, 16), (257, 17), (48, 48), (2, 2), (515, 33), (1000, 64)]
    case = PagedCase(torch.bfloat16, heads, kv_heads, dim, page, seqs, window, seed=dim + 5)
    assert ops.prefill_block_rows(dim, heads, kv_heads) == 32
    work = shared_out_work(case, seqs, window, shares)
    assert work.slots >= 4
    out = torch.zeros(case.qsl[-1], heads * dim, dtype=torch.bfloat16, device=DEV)
    ops.attention_prefill(
        out, case.dev(case.q), heads * dim, case.dev(case.kp), case.dev(case.vp), case.dev(case.table),
        case.ints(case.qsl), case.ints([c for c, _ in seqs]), work, heads, dim ** -0.5, window,
        max(c for c, _ in seqs), 32,
    )
    torch.testing.assert_close(out.float().cpu(), case.expected, **tol(torch.bfloat16))


def test_attention_prefill_mfma_shares_by_the_planner(ops, monkeypatch):
    """The work lists :meth:`Ops.prefill_blocks` makes itself: a short portion at the end of a
    long context beside another request's (every long block shared out several times) with a far
    key that carries the result, a prompt of 5,000 tokens on one KV head (a quarter of the
    workgroups: long shares), and prompts that fill the device or are short (nothing shared
    out); each against the plain attention."""
    heads, kv_heads, dim, page = 28, 4, 128, 16
    for seqs, spike, shared in (([(6000, 96), (300, 40)], 77, True), ([(2048, 2048)], None, False),
                                ([(500, 500), (90, 90)], None, False), ([(5000, 5000)], None, True)):
        if seqs[0][0] == 5000:
            heads, kv_heads = 7, 1  # (and the plain attention on the host takes a quarter of the time)
        case = PagedCase(torch.bfloat16, heads, kv_heads, dim, page, seqs, None, seed=21, spike=spike)
        work = ops.prefill_blocks([q for _, q in seqs], [c for c, _ in seqs], 32, heads=heads, kv_heads=kv_heads,
                                  head_dim=dim, block_size=page)
        assert (work.ranges is not None) == shared, seqs
        out = torch.zeros(case.qsl[-1], heads * dim, dtype=torch.bfloat16, device=DEV)
        ops.attention_prefill(
            out, case.dev(case.q), heads * dim, case.dev(case.kp), case.dev(case.vp), case.dev(case.table),
            case.ints(case.qsl), case.ints([c for c, _ in seqs]), work, heads, dim ** -0.5, None, max(c for c, _ in seqs), 32,
        )
        torch.testing.assert_close(out.float().cpu(), case.expected, **tol(torch.bfloat16))
        if spike is not None:
            assert float(case.expected[:96].abs().mean()) > 4.0


def test_attention_prefill_mfma_far_key(ops):
    heads, kv_heads, dim, page = 28, 4, 128, 16
    seqs = [(3000, 40), (2100, 2100)]
    case = PagedCase(torch.bfloat16, heads, kv_heads, dim, page, seqs, None, seed=11, spike=77)
    rows, blocks = prefill_blocks_of(ops, case, heads, kv_heads, dim, seqs)
    out = torch.zeros(case.qsl[-1], heads * dim, dtype=torch.bfloat16, device=DEV)
    ops.attention_prefill(
        out, case.dev(case.q), heads * dim, case.dev(case.kp), case.dev(case.vp), case.dev(case.table),
        case.ints(case.qsl), case.ints([c for c, _ in seqs]), case.ints(blocks), heads, dim ** -0.5, None, 3000, rows,
    )
    got = out.float().cpu()
    torch.testing.assert_close(got, case.expected, **tol(torch.bfloat16))
    assert float(case.expected[:40].abs().mean()) > 4.0


@pytest.mark.parametrize("heads,kv_heads,dim,page", [(14, 2, 128, 16), (3, 1, 32, 8)])
@pytest.mark.parametrize("window", [40, 64, 97])
def test_attention_at_the_windows_edge(ops, heads, kv_heads, dim, page, window):
    """One key that would carry the result lies just outside the window of a single-token
    request's query, then just inside; and inside the window of some rows of a prompt portion
    and outside that of others.  A kernel that is one key off at either edge returns that key's
    value (5.0) where the plain attention does not, or the other way round."""
    ctx = 300
    for spike, carried in ((ctx - 1 - window, False), (ctx - window, True), (ctx - 1, True)):
        case = PagedCase(torch.bfloat16, heads, kv_heads, dim, page, [(ctx, 1)], window, seed=spike, spike=spike)
        assert (float(case.expected.abs().mean()) > 4.0) == carried
        out = torch.zeros(1, heads * dim, dtype=torch.bfloat16, device=DEV)
        ops.attention_decode(
            out, case.dev(case.q), heads * dim, case.dev(case.kp), case.dev(case.vp), case.dev(case.table),
            case.ints(case.qsl), case.ints([ctx]), 0, 1, heads, dim ** -0.5, window, ctx,
        )
        torch.testing.assert_close(out.float().cpu(), case.expected, **tol(torch.bfloat16))
        for dtype in (torch.float32, torch.bfloat16):
            exact = PagedCase(dtype, heads, kv_heads, dim, page, [(ctx, 1)], window, seed=spike, spike=spike)
            got = ops.paged_attention_generic(
                exact.dev(exact.q), heads * dim, exact.dev(exact.kp), exact.dev(exact.vp), exact.dev(exact.table),
                exact.ints(exact.token_seq), exact.ints(exact.positions), heads, dim ** -0.5, window,
            ).float().cpu()
            torch.testing.assert_close(got, exact.expected, **tol(dtype))
    # a portion of 70 rows (positions 230..299): the key at 250 is seen by rows 250 .. 249 + window
    # only, so some rows of one 16-row block see it and others do not, at both edges
    qlen, spike = 70, 250
    case = PagedCase(torch.bfloat16, heads, kv_heads, dim, page, [(ctx, qlen)], window, seed=7, spike=spike)
    rows = case.expected.view(qlen, -1).abs().mean(1) > 4.0
    positions = torch.arange(ctx - qlen, ctx)
    assert torch.equal(rows, (positions >= spike) & (positions <= spike + window - 1))
    rows, blocks = prefill_blocks_of(ops, case, heads, kv_heads, dim, [(ctx, qlen)])
    out = torch.zeros(qlen, heads * dim, dtype=torch.bfloat16, device=DEV)
    ops.attention_prefill(
        out, case.dev(case.q), heads * dim, case.dev(case.kp), case.dev(case.vp), case.dev(case.table),
        case.ints(case.qsl), case.ints([ctx]), case.ints(blocks), heads, dim ** -0.5, window, ctx, rows,
    )
    torch.testing.assert_close(out.float().cpu(), case.expected, **tol(torch.bfloat16))
    got = ops.paged_attention_generic(
        case.dev(case.q), heads * dim, case.dev(case.kp), case.dev(case.vp), case.dev(case.table),
        case.ints(case.token_seq), case.ints(case.positions), heads, dim ** -0.5, window,
    ).float().cpu()
    torch.testing.assert_close(got, case.expected, **tol(torch.bfloat16))


# -- sampling ---------------------------------------------------------------------------------------


def test_argmax_lowest_index_of_ties(ops):
    logits = torch.zeros(3, 152064)
    logits[0, 77] = 1.0
    logits[0, 151000] = 1.0
    logits[1, 152063] = 2.0
    got = ops.argmax(logits.to(DEV)).cpu().tolist()
    assert got == [77, 152063, 0]


def sample_rows(ops, logits, params, seeds, draws, histories=None):
    from turboserve_amd.sampling.sampler import Sampler

    return Sampler(ops).sample(logits.to(DEV), params, seeds, draws, histories)


@pytest.mark.parametrize("vocab", [320, 5003])
def test_sampler_stages_against_plain(ops, vocab):
    """Every stage alone and combined, row by row against the plain implementation: the chosen
    token's cumulative interval (64-bit) contains the row's uniform number."""
    from turboserve_amd.sampling.params import SamplingParams

    g = torch.Generator().manual_seed(vocab)
    settings = [
        dict(temperature=0.0),
        dict(temperature=0.0, repetition_penalty=1.7),
        dict(temperature=0.7),
        dict(temperature=1.3, top_k=5),
        dict(temperature=1.0, top_p=0.6),
        dict(temperature=0.9, top_k=40, top_p=0.8, repetition_penalty=1.3),
        dict(temperature=1.0, top_k=1),
        dict(temperature=1e-3),
    ]
    rows = len(settings) * 4
    logits = torch.randn(rows, vocab, generator=g) * 3
    params = [SamplingParams(logprobs=True, **settings[i % len(settings)]) for i in range(rows)]
    seeds = [1000 + i * 7919 + (i << 40) for i in range(rows)]
    draws = [i * 3 for i in range(rows)]
    histories = [torch.randint(0, vocab, (20,), generator=g).tolist() for _ in range(rows)]
    out = sample_rows(ops, logits, params, seeds, draws, histories)
    for i, p in enumerate(params):
        token = out.token_ids[i]
        want, cdf = plain.sample_token(
            logits[i], temperature=p.temperature, seed=seeds[i], draw_index=draws[i], top_k=p.top_k, top_p=p.top_p,
            penalty=p.repetition_penalty, history=histories[i],
        )
        penalised = plain.repetition_penalty(logits[i], histories[i], p.repetition_penalty)
        assert abs(out.logprobs[i] - plain.log_softmax_at(penalised, token)) < 1e-4, f"row {i} logprob"
        if p.temperature == 0.0:
            assert token == want, f"row {i} {settings[i % len(settings)]}"
            continue
        u = plain.philox_uniform(seeds[i], draws[i])
        low = float(cdf[token - 1]) if token > 0 else 0.0
        high = float(cdf[token])
        assert high > low, f"row {i}: token {token} has no mass after {settings[i % len(settings)]}"
        assert low - 1e-5 <= u <= high + 1e-5, f"row {i} {settings[i % len(settings)]}: u={u} not in [{low}, {high}]"


def kept_after_truncation(logits: torch.Tensor, temperature: float, top_k: int, top_p: float) -> torch.Tensor:
    """The plain truncation rules (``plain.top_k_filter``, ``plain.top_p_filter``) for a long row:
    the same sets, found with a sort and cumulative sums instead of a loop over the vocabulary."""
    work = logits.double() / temperature
    keep = torch.ones_like(work, dtype=torch.bool)
    if 0 < top_k < work.numel():
        keep = work >= torch.sort(work, descending=True).values[top_k - 1]
    if top_p < 1.0:
        filtered = work.masked_fill(~keep, float("-inf"))
        probs = torch.softmax(filtered, dim=-1)
        values, inverse = torch.unique(filtered, sorted=True, return_inverse=True)
        per_value = torch.zeros(values.numel(), dtype=torch.float64).index_add_(0, inverse, probs)
        above = per_value.sum() - torch.cumsum(per_value, dim=0)  # mass strictly above each distinct value
        keep = keep & (above[inverse] <= top_p)
    return keep


def test_truncation_helper_is_the_plain_rule():
    g = torch.Generator().manual_seed(9)
    for quantum in (None, 0.5):
        logits = torch.randn(300, generator=g) * 3
        if quantum:
            logits = torch.round(logits / quantum) * quantum  # many equal values
        for top_k, top_p in ((0, 0.7), (7, 1.0), (20, 0.5), (3, 0.9)):
            want = torch.isfinite(plain.top_p_filter(plain.top_k_filter(logits / 0.8, top_k), top_p))
            assert torch.equal(kept_after_truncation(logits, 0.8, top_k, top_p), want)


@pytest.mark.parametrize("vocab", [152064, 40001])
def test_sampler_on_a_long_row_with_equal_logits(ops, vocab):
    """A vocabulary of real size (rows that are and are not 16-byte aligned), smooth logits,
    logits on a grid of 0.25 (thousands of equal values, keys whose low bits are zero) and peaked
    rows (the kernel's short way through a list of the likely tokens): the token lies in what the
    plain truncation keeps, and its cumulative interval holds the uniform number."""
    from turboserve_amd.sampling.params import SamplingParams

    g = torch.Generator().manual_seed(vocab)
    settings = [dict(temperature=0.8), dict(temperature=0.8, top_k=50, top_p=0.9), dict(temperature=1.0, top_p=0.6),
                dict(temperature=1.3, top_k=5), dict(temperature=0.7, top_k=2000, top_p=0.95), dict(temperature=1.0, top_p=0.05)]
    group = 2 * len(settings)
    rows = 5 * group
    logits = torch.randn(rows, vocab, generator=g) * 2.5
    logits[group:2 * group] = torch.round(logits[group:2 * group] * 4) / 4
    # Rows as a language model makes them, which the kernel's short way takes (few tokens far above
    # the rest): thirty likely tokens all over the vocabulary; the same on a grid of 0.25 (equal
    # logits among the likely ones); fifty likely tokens at the start of the vocabulary (one
    # wavefront lists them all) with every logit negative.
    for i in range(2 * group, 4 * group):
        spots = torch.randperm(vocab, generator=g)[:30]
        logits[i, spots] = torch.rand(30, generator=g) * 12 + 12
    logits[3 * group:4 * group] = torch.round(logits[3 * group:4 * group] * 4) / 4
    logits[4 * group:] = logits[4 * group:] - 40.0
    logits[4 * group:, :50] += torch.rand(group, 50, generator=g) * 10 + 12
    assert float(logits[4 * group:].max()) < 0
    params = [SamplingParams(**settings[i % len(settings)]) for i in range(rows)]
    seeds = [77 + i * 104729 for i in range(rows)]
    draws = [i for i in range(rows)]
    out = sample_rows(ops, logits, params, seeds, draws)
    for i, p in enumerate(params):
        token = out.token_ids[i]
        keep = kept_after_truncation(logits[i], p.temperature, p.top_k, p.top_p)
        assert bool(keep[token]), f"row {i} {settings[i % len(settings)]}: token {token} is outside the kept set of {int(keep.sum())}"
        probs = torch.softmax((logits[i].double() / p.temperature).masked_fill(~keep, float("-inf")), dim=-1)
        cdf = torch.cumsum(probs, dim=-1)
        u = plain.philox_uniform(seeds[i], draws[i])
        low = float(cdf[token - 1]) if token > 0 else 0.0
        assert low - 1e-5 <= u <= float(cdf[token]) + 1e-5, f"row {i}: u={u} not in [{low}, {float(cdf[token])}]"


def test_samplers_short_and_long_way_choose_alike(ops):
    """The sampling kernel's short way (a list of the likely tokens) and its long way (the whole
    row) use the same integer masses and comparisons: on thousands of peaked rows of every
    truncation they choose the same token, but for a draw that falls within rounding of an
    interval's end (the two add the same masses up in different orders)."""
    from turboserve_amd.kernels.ops import Ops
    from turboserve_amd.sampling.params import SamplingParams

    long_way = Ops(DEV)
    long_way.sample_max_listed = 0
    g = torch.Generator().manual_seed(12)
    settings = [dict(temperature=0.7, top_k=20, top_p=0.8), dict(temperature=1.0, top_k=50), dict(temperature=0.9, top_p=0.9),
                dict(temperature=1.2, top_k=3, top_p=0.5), dict(temperature=0.8, top_k=400, top_p=0.95),
                dict(temperature=0.6, top_p=0.3, repetition_penalty=1.3)]
    differing = 0
    for vocab, rows in ((5003, 3000), (152064, 96)):
        logits = torch.randn(rows, vocab, generator=g) * 2.5
        for i in range(rows):
            spots = torch.randperm(vocab, generator=g)[:1 + i % 40]
            logits[i, spots] = torch.rand(spots.numel(), generator=g) * 12 + 10
        logits[::3] = torch.round(logits[::3] * 8) / 8  # equal logits among the likely ones
        params = [SamplingParams(**settings[i % len(settings)]) for i in range(rows)]
        seeds = [11 + 7919 * i for i in range(rows)]
        draws = [i % 17 for i in range(rows)]
        histories = [torch.randint(0, vocab, (30,), generator=g).tolist() for _ in range(rows)]
        short = sample_rows(ops, logits, params, seeds, draws, histories).token_ids
        long = sample_rows(long_way, logits, params, seeds, draws, histories).token_ids
        differing += sum(a != b for a, b in zip(short, long))
    assert differing <= 2, f"{differing} rows differ"


def test_sampler_keeps_equal_logits_together(ops):
    """Five equal logits at the edge of top-k 3 are all kept (the plain rule: below the k-th
    largest is cut) and all drawn; a nucleus that ends inside a group of equal logits keeps the group."""
    from turboserve_amd.sampling.params import SamplingParams

    logits = torch.full((1, 64), -4.0)
    logits[0, [3, 9]] = 2.0
    logits[0, [11, 20, 31, 40, 63]] = 1.0  # the third largest value, five times
    many = logits.repeat(600, 1)
    out = sample_rows(ops, many, [SamplingParams(temperature=1.0, top_k=3)] * 600, [5] * 600, list(range(600)))
    assert set(out.token_ids) == {3, 9, 11, 20, 31, 40, 63}
    # mass above the 1.0 group is 2 e^2 / (2 e^2 + 5 e + 57 e^-4) = 0.5024 <= 0.6: the group stays; 0.5 cuts it
    out = sample_rows(ops, many, [SamplingParams(temperature=1.0, top_p=0.6)] * 600, [6] * 600, list(range(600)))
    assert set(out.token_ids) == {3, 9, 11, 20, 31, 40, 63}
    out = sample_rows(ops, many, [SamplingParams(temperature=1.0, top_p=0.5)] * 600, [7] * 600, list(range(600)))
    assert set(out.token_ids) == {3, 9}


def test_sampler_rows_are_independent(ops):
    """A batch equals its rows one by one, and a row does not depend on its neighbours
    (tests/unit/test_sampler.py:131-149, 198-215)."""
    from turboserve_amd.sampling.params import SamplingParams

    g = torch.Generator().manual_seed(1)
    logits = torch.randn(6, 777, generator=g)
    params = [SamplingParams(temperature=t, top_k=k) for t, k in ((1.0, 0), (0.0, 0), (0.5, 10), (2.0, 0), (1.0, 3), (0.0, 5))]
    seeds, draws = [5, 6, 7, 8, 9, 10], [0, 1, 2, 3, 4, 5]
    batch = sample_rows(ops, logits, params, seeds, draws).token_ids
    single = [sample_rows(ops, logits[i:i + 1], params[i:i + 1], seeds[i:i + 1], draws[i:i + 1]).token_ids[0] for i in range(6)]
    assert batch == single
    assert batch[1] == int(logits[1].argmax()) and batch[5] == int(logits[5].argmax())  # greedy ignores top-k


def test_sampler_distribution(ops):
    """Draws follow the softmax: 4000 counters of one seed against the probabilities."""
    from turboserve_amd.sampling.params import SamplingParams

    logits = torch.tensor([[2.0, 1.0, 0.0, -1.0, 0.5]]).repeat(4000, 1)
    out = sample_rows(ops, logits, [SamplingParams(temperature=1.0)] * 4000, [42] * 4000, list(range(4000)))
    counts = torch.bincount(torch.tensor(out.token_ids), minlength=5).float() / 4000
    probs = torch.softmax(logits[0], -1)
    assert float((counts - probs).abs().max()) < 0.03
    top2 = sample_rows(ops, logits[:500], [SamplingParams(temperature=1.0, top_k=2)] * 500, [1] * 500, list(range(500)))
    assert set(top2.token_ids) == {0, 1}  # the support of top-k (tests/unit/test_sampler.py:121-128)


def test_philox_matches_plain(ops):
    """The kernel's uniform numbers are the plain implementation's: with logits that make the
    cumulative distribution a ruler, the drawn token reads off u."""
    from turboserve_amd.sampling.params import SamplingParams

    vocab = 4096
    logits = torch.zeros(64, vocab)
    seeds = [random.Random(i).getrandbits(64) for i in range(64)]
    draws = [random.Random(100 + i).getrandbits(31) for i in range(64)]
    out = sample_rows(ops, logits, [SamplingParams(temperature=1.0)] * 64, seeds, draws)
    for token, seed, draw in zip(out.token_ids, seeds, draws):
        assert abs(token - int(plain.philox_uniform(seed, draw) * vocab)) <= 1
