"""Each kernel alone against the plain implementation's function of the same
operation, at sizes other than the engine's tiny models: widths and
vocabularies that are no power of two, odd group sizes, head sizes in steps
of 16, pages of several sizes."""
import numpy as np
import pytest
import torch

from plain import model as pm
from plain import sampler as ps
from alofa_amd.errors import AlofaError

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def ops():
    from alofa_amd import ops as o
    return o


def t(a, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV).to(dtype)


def bf(a):
    """Round a float32 array to bfloat16 and back: what the bfloat16 kernels are given."""
    return torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16).float().numpy()


def close(got, ref, rel, what=""):
    got = got.detach().float().cpu().numpy() if isinstance(got, torch.Tensor) else got
    err = np.abs(got.astype(np.float64) - ref.astype(np.float64)).max()
    b = rel * max(1.0, float(np.abs(ref).max()))
    assert np.isfinite(got).all() and err <= b, f"{what}: {err:.3e} > {b:.3e}"


EXACT, BF16 = 1e-6, 1e-2     # exact kernels round where the plain code rounds; bfloat16 outputs carry 8 bits


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed_gather(dtype):
    rng = np.random.default_rng(0)
    table = bf(rng.standard_normal((331, 72)).astype(np.float32))
    ids = rng.integers(0, 331, 19)
    out = torch.empty(19, 72, device=DEV)
    ops().embed_gather(out, t(table, dtype), t(ids.astype(np.int32), torch.int32))
    assert np.array_equal(out.cpu().numpy(), pm.embed(table, ids))


@pytest.mark.parametrize("width", [80, 896, 1000, 1024, 1026, 2044, 3584, 5120, 8192, 9000])     # rows kept in registers (multiples of four up to 8,192) and rows read twice
def test_rmsnorm(width):
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((9, width)) * 3).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(width)).astype(np.float32)
    out = torch.empty(9, width, device=DEV)
    ops().rmsnorm(out, t(x), t(w), 1e-5, True)
    close(out, pm.rmsnorm(x, w, 1e-5), EXACT, "exact")
    outb = torch.empty(9, width, device=DEV, dtype=torch.bfloat16)
    ops().rmsnorm(outb, t(x), t(w), 1e-5, False)
    close(outb, pm.rmsnorm(x, w, 1e-5), BF16, "bf16")
    rows = np.array([8, 0, 3, 3], dtype=np.int32)                       # with the row gather
    outg = torch.empty(4, width, device=DEV)
    ops().rmsnorm(outg, t(x), t(w), 1e-5, True, t(rows, torch.int32))
    close(outg, pm.rmsnorm(x[rows], w, 1e-5), EXACT, "gather")
    outgb = torch.empty(4, width, device=DEV, dtype=torch.bfloat16)
    ops().rmsnorm(outgb, t(x), t(w), 1e-5, False, t(rows, torch.int32))
    close(outgb, pm.rmsnorm(x[rows], w, 1e-5), BF16, "bf16 gather")


SHAPES = [(1, 100, 72), (5, 130, 200), (70, 33, 264), (130, 257, 48), (3, 64, 1000), (300, 200, 136), (64, 300, 96), (65, 129, 40)]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_gemm_exact(M, N, K):
    rng = np.random.default_rng(2)
    a = rng.standard_normal((M, K)).astype(np.float32)
    w = rng.standard_normal((N, K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    out = torch.empty(M, N, device=DEV)
    ops().gemm(out, t(a), t(w), t(b), exact=True)
    close(out, pm.linear(a, w, b), EXACT, "bias")
    res = rng.standard_normal((M, N)).astype(np.float32)
    acc = t(res)
    ops().gemm(acc, t(a), t(w), add_to_out=True, exact=True)
    close(acc, pm.add(res, pm.linear(a, w)), EXACT, "residual")
    # a row's result does not depend on what else is in the batch
    one = torch.empty(1, N, device=DEV)
    ops().gemm(one, t(a[M - 1:]), t(w), t(b), exact=True)
    assert torch.equal(one[0], out[M - 1])


# shapes whose few tiles make the tiled kernel share K out among blocks as well
DEEP_SHAPES = [(40, 130, 1000), (9, 64, 4864), (130, 200, 2056), (64, 896, 672), (3, 33000, 72), (50, 40011, 40)]   # the last two: a long matrix, 64-row tiles


def with_kernels(shapes):
    """Every shape with each bfloat16 product that takes it (the streaming kernel: at most 64 rows)."""
    return [(*shape, kernel) for shape in shapes for kernel in ("stream", "tiled") if kernel == "tiled" or shape[0] <= 64]


@pytest.mark.parametrize("M,N,K,kernel", with_kernels(SHAPES + DEEP_SHAPES))
def test_gemm_bf16(M, N, K, kernel):
    rng = np.random.default_rng(3)
    a, w = bf(rng.standard_normal((M, K)).astype(np.float32)), bf(rng.standard_normal((N, K)).astype(np.float32) * 0.1)
    b = rng.standard_normal(N).astype(np.float32)
    out = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    ops().gemm(out, t(a, torch.bfloat16), t(w, torch.bfloat16), t(b), kernel=kernel)
    close(out, pm.linear(a, w, b), BF16, "bf16 out")
    outf = torch.empty(M, N, device=DEV)
    ops().gemm(outf, t(a, torch.bfloat16), t(w, torch.bfloat16), kernel=kernel)
    close(outf, pm.linear(a, w), 1e-4, "f32 out")
    res = rng.standard_normal((M, N)).astype(np.float32)
    acc = t(res)
    ops().gemm(acc, t(a, torch.bfloat16), t(w, torch.bfloat16), add_to_out=True, kernel=kernel)
    close(acc, pm.add(res, pm.linear(a, w)), 1e-4, "residual")
    if kernel == "tiled":
        return
    # a weight stored in float32 stays float32 and is multiplied as such
    outw = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    w32 = rng.standard_normal((N, K)).astype(np.float32) * 0.1
    ops().gemm(outw, t(a, torch.bfloat16), t(w32), t(b))
    close(outw, pm.linear(a, w32, b), BF16, "f32 weight")


@pytest.mark.parametrize("M,N,K", [(1, 1152, 896), (8, 1152, 896), (16, 130, 264), (3, 97, 80), (11, 200, 2040), (16, 176, 1000), (7, 3000, 8192), (5, 4608, 3584), (17, 64, 64), (8, 9000, 8192)])
def test_product_that_takes_the_norm_with_it(M, N, K):
    """The streaming product applies the RMSNorm of its float32 rows on the way (x * w rounded to
    bfloat16 as the operand, the row's factor on the finished sum): against the plain norm followed
    by the plain product, and against the two kernels run one after the other."""
    o = ops()
    rng = np.random.default_rng(8)
    x = (rng.standard_normal((M, K)) * rng.uniform(0.05, 30.0, (M, 1))).astype(np.float32)     # rows of very different size
    nw = (1.0 + 0.3 * rng.standard_normal(K)).astype(np.float32)
    w, w2 = (bf(rng.standard_normal((N, K)).astype(np.float32) * 0.1) for _ in range(2))
    b = rng.standard_normal(N).astype(np.float32)
    eps = 1e-5
    if not o.can_fuse_norm(M, t(w, torch.bfloat16), torch.bfloat16):
        from alofa_amd.csrc.build import load
        assert (M > 16 or load().alofa_gemm_skinny_splits(1, M, N, K, 0) > 1 or o.few_rows_kernel(M, N, K) != "stream"), \
            "only a product that has more than 16 rows, shares K out over blocks or is the tiled kernel's may refuse"
        with pytest.raises(AlofaError):
            o.gemm(torch.empty(M, N, device=DEV, dtype=torch.bfloat16), t(x), t(w, torch.bfloat16), t(b), norm=(t(nw), eps))
        return
    normed = pm.rmsnorm(x, nw, eps)
    out = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    o.gemm(out, t(x), t(w, torch.bfloat16), t(b), norm=(t(nw), eps))
    close(out, pm.linear(normed, w, b), BF16, "norm + product + bias")
    # the two kernels one after the other: the same up to the rounding of the normed rows
    y = torch.empty(M, K, device=DEV, dtype=torch.bfloat16)
    o.rmsnorm(y, t(x), t(nw), eps, False)
    two = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    o.gemm(two, y, t(w, torch.bfloat16), t(b), kernel="stream")
    assert (out.float() - two.float()).abs().max().item() <= 2e-2 * max(1.0, two.float().abs().max().item())
    # rows do not depend on their neighbours: the first row alone gives the same bits (where the same kernel takes one row)
    one = torch.empty(1, N, device=DEV, dtype=torch.bfloat16)
    o.gemm(one, t(x[:1]), t(w, torch.bfloat16), t(b), norm=(t(nw), eps), kernel=o.few_rows_kernel(M, N, K, normed=True))
    assert torch.equal(one[0], out[0])
    assert o.can_fuse_norm(M, t(w, torch.bfloat16), torch.bfloat16, swiglu=True)
    act = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    o.gemm_swiglu(act, t(x), t(w, torch.bfloat16), t(w2, torch.bfloat16), norm=(t(nw), eps))
    close(act, pm.swiglu(pm.linear(normed, w), pm.linear(normed, w2)), BF16, "norm + gate/up + swiglu")


@pytest.mark.parametrize("M,N,K", [(65, 896, 4864), (200, 896, 4864), (1030, 896, 4864), (2048, 896, 4864), (64, 3584, 3584), (40, 3584, 18944), (17, 1536, 8960),
                                   (300, 3584, 18944), (64, 896, 896), (2048, 896, 896), (8, 896, 4864), (130, 1000, 3200), (256, 5120, 5120)])
def test_norm_behind_a_product_that_adds_to_the_residual_stream(M, N, K):
    """``gemm(..., add_to_out=True, then_norm=)``: the residual stream's new rows and their RMSNorm. Where the product
    shares K out among blocks and a second launch adds the shares (long K, few tiles), that launch has whole rows in
    hand and normalises them on its way; everywhere else the norm kernel runs behind the product. Either way the
    values are those of the product followed by the norm kernel, bit for bit."""
    o = ops()
    rng = np.random.default_rng(73)
    scale = rng.uniform(0.05, 30.0, (M, 1))
    resid = (rng.standard_normal((M, N)) * scale).astype(np.float32)
    a = bf((rng.standard_normal((M, K)) * scale).astype(np.float32))
    w = bf(rng.standard_normal((N, K)).astype(np.float32) * 0.1)
    nw, eps = (1.0 + 0.3 * rng.standard_normal(N)).astype(np.float32), 1e-5
    at, wt, nwt = t(a, torch.bfloat16), t(w, torch.bfloat16), t(nw)
    plain, sep = t(resid), torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    o.gemm(plain, at, wt, add_to_out=True)
    o.rmsnorm(sep, plain, nwt, eps, False)
    out, rows = t(resid), torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
    o.gemm(out, at, wt, add_to_out=True, then_norm=(nwt, eps, rows))
    assert torch.equal(out, plain) and torch.equal(rows, sep)
    x = resid.astype(np.float64) + a.astype(np.float64) @ w.astype(np.float64).T
    close(rows, pm.rmsnorm(x.astype(np.float32), nw, eps), BF16, "the norm of the new rows")
    # float32 rows for the exact path: the norm kernel behind the exact product
    exact_out, exact_rows = t(resid), torch.empty(M, N, device=DEV)
    if M <= 300:
        o.gemm(exact_out, t(a), t(w), add_to_out=True, exact=True, then_norm=(nwt, eps, exact_rows))
        close(exact_rows, pm.rmsnorm(x.astype(np.float32), nw, eps), 2e-6, "exact")
    with pytest.raises(AlofaError):
        o.gemm(torch.empty(M, N, device=DEV, dtype=torch.bfloat16), at, wt, then_norm=(nwt, eps, rows))       # not the residual stream


@pytest.mark.parametrize("M,N,K", [(1, 1152, 896), (8, 896, 4864), (3, 97, 80), (7, 1000, 1544), (5, 130, 6144), (2, 64, 8), (4, 4864, 896), (6, 35, 520)])
def test_product_for_very_few_rows(M, N, K):
    """The vector-unit product for at most eight rows, every form of it (store with bias, float32 store,
    residual, gate/up, and the norm on the way in), at sizes that end inside a run of 512 along K and
    inside a block's columns; a row's bits do not depend on the rows beside it."""
    o = ops()
    rng = np.random.default_rng(44)
    a, w, w2 = (bf(rng.standard_normal(shape).astype(np.float32) * scale) for shape, scale in (((M, K), 1.0), ((N, K), 0.1), ((N, K), 0.1)))
    b = rng.standard_normal(N).astype(np.float32)
    at, wt, w2t = t(a, torch.bfloat16), t(w, torch.bfloat16), t(w2, torch.bfloat16)
    out = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    o.gemm(out, at, wt, t(b), kernel="rows")
    close(out, pm.linear(a, w, b), BF16, "store + bias")
    outf = torch.empty(M, N, device=DEV)
    o.gemm(outf, at, wt, kernel="rows")
    close(outf, pm.linear(a, w), 1e-4, "float32 store")
    res = rng.standard_normal((M, N)).astype(np.float32)
    acc = t(res)
    o.gemm(acc, at, wt, add_to_out=True, kernel="rows")
    close(acc, pm.add(res, pm.linear(a, w)), 1e-4, "residual")
    act = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    o.gemm_swiglu(act, at, wt, w2t, kernel="rows")
    close(act, pm.swiglu(pm.linear(a, w), pm.linear(a, w2)), BF16, "gate/up")
    # float32 rows that take a norm on their way
    x = (rng.standard_normal((M, K)) * rng.uniform(0.05, 30.0, (M, 1))).astype(np.float32)
    nw = (1.0 + 0.3 * rng.standard_normal(K)).astype(np.float32)
    normed = pm.rmsnorm(x, nw, 1e-5)
    outn, actn = torch.empty(M, N, device=DEV, dtype=torch.bfloat16), torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    o.gemm(outn, t(x), wt, t(b), norm=(t(nw), 1e-5), kernel="rows")
    close(outn, pm.linear(normed, w, b), BF16, "norm + store + bias")
    o.gemm_swiglu(actn, t(x), wt, w2t, norm=(t(nw), 1e-5), kernel="rows")
    close(actn, pm.swiglu(pm.linear(normed, w), pm.linear(normed, w2)), BF16, "norm + gate/up")
    # the last row alone: the same bits in every form
    r = M - 1
    one, onef, one_acc, one_act, one_n = (torch.empty(1, N, device=DEV, dtype=d) for d in (torch.bfloat16, torch.float32, torch.float32, torch.bfloat16, torch.bfloat16))
    o.gemm(one, at[r:], wt, t(b), kernel="rows")
    o.gemm(onef, at[r:], wt, kernel="rows")
    one_acc.copy_(t(res[r:]))
    o.gemm(one_acc, at[r:], wt, add_to_out=True, kernel="rows")
    o.gemm_swiglu(one_act, at[r:], wt, w2t, kernel="rows")
    o.gemm(one_n, t(x[r:]), wt, t(b), norm=(t(nw), 1e-5), kernel="rows")
    for alone, batch, what in ((one, out, "store"), (onef, outf, "float32 store"), (one_acc, acc, "residual"), (one_act, act, "gate/up"), (one_n, outn, "norm + store")):
        assert torch.equal(alone[0], batch[r]), what


def test_product_for_very_few_rows_refuses_what_it_cannot_take():
    o = ops()
    w = torch.zeros(16, 6152, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(AlofaError):          # more rows than sixteen
        o.gemm(torch.empty(17, 16, device=DEV), torch.zeros(17, 64, device=DEV, dtype=torch.bfloat16), w[:, :64].contiguous(), kernel="rows")
    with pytest.raises(AlofaError):          # more than eight: plain products only
        o.gemm_swiglu(torch.empty(9, 16, device=DEV, dtype=torch.bfloat16), torch.zeros(9, 64, device=DEV, dtype=torch.bfloat16), w[:, :64].contiguous(), w[:, :64].contiguous(), kernel="rows")
    with pytest.raises(AlofaError):          # ... of rows that its waves cover at once
        o.gemm(torch.empty(9, 16, device=DEV), torch.zeros(9, 6152, device=DEV, dtype=torch.bfloat16), w, kernel="rows")
    with pytest.raises(AlofaError):          # rows longer than its waves cover at once: plain products only, not gate/up
        o.gemm_swiglu(torch.empty(2, 16, device=DEV, dtype=torch.bfloat16), torch.zeros(2, 6152, device=DEV, dtype=torch.bfloat16), w, w, kernel="rows")
    with pytest.raises(AlofaError):          # ... and not with a norm on the way
        o.gemm(torch.empty(2, 16, device=DEV, dtype=torch.bfloat16), torch.zeros(2, 6152, device=DEV), w, norm=(torch.ones(6152, device=DEV), 1e-5), kernel="rows")
    from alofa_amd.csrc.build import load
    fits = load().alofa_gemm_rows_fits
    assert fits(8, 16, 6144, 0) == 1 and fits(8, 16, 6152, 0) == 0 and fits(8, 16, 6152, 1) == 1 and fits(9, 16, 64, 0) == 0 and fits(16, 16, 64, 1) == 1 and fits(17, 16, 64, 1) == 0 and fits(9, 16, 6152, 1) == 0


@pytest.mark.parametrize("M,N,K", [(1, 130, 18944), (4, 67, 6152), (8, 96, 12296), (3, 40, 27648), (9, 35, 520), (12, 896, 4864), (16, 130, 1544)])
def test_product_for_very_few_rows_against_long_rows(M, N, K):
    """The plain forms (store with bias, float32 store, residual) beyond what every form takes: K beyond the runs
    that the waves of a block cover at once (the kernel that loops over them, at lengths that end inside a run
    and inside a round of the waves), and nine to sixteen rows; a row's bits do not depend on the rows beside it."""
    o = ops()
    rng = np.random.default_rng(45)
    a, w = bf(rng.standard_normal((M, K)).astype(np.float32)), bf(rng.standard_normal((N, K)).astype(np.float32) * 0.1)
    b = rng.standard_normal(N).astype(np.float32)
    at, wt = t(a, torch.bfloat16), t(w, torch.bfloat16)
    out = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    o.gemm(out, at, wt, t(b), kernel="rows")
    close(out, pm.linear(a, w, b), BF16, "store + bias")
    outf = torch.empty(M, N, device=DEV)
    o.gemm(outf, at, wt, kernel="rows")
    close(outf, pm.linear(a, w), 2e-4, "float32 store")
    res = rng.standard_normal((M, N)).astype(np.float32)
    acc = t(res)
    o.gemm(acc, at, wt, add_to_out=True, kernel="rows")
    close(acc, pm.add(res, pm.linear(a, w)), 2e-4, "residual")
    onef = torch.empty(1, N, device=DEV)
    o.gemm(onef, at[M - 1:], wt, kernel="rows")
    assert torch.equal(onef[0], outf[M - 1])


def test_gemm_split_over_blocks_is_repeatable():
    """Few rows and few columns: K is split over blocks that hand partial sums to the last one
    to arrive. The additions are in a fixed order, so every run gives the same bits; a partial
    sum that was not yet in memory when it was read would show as a difference. Two products
    of different shapes alternate, so that what the workspace held before is never the answer."""
    rng = np.random.default_rng(40)
    cases = []
    from alofa_amd.csrc.build import load
    for M, N, K, kernel in [(3, 1082, 4032, "stream"), (40, 864, 1344, "stream"), (5, 672, 4864, "stream"), (2, 144, 8192, "stream"),
                            (40, 864, 672, "tiled"), (150, 672, 4864, "tiled"), (20, 144, 2048, "tiled")]:
        # (the product for few rows shares K out where a block would otherwise read much: these shapes are such)
        assert kernel != "stream" or load().alofa_gemm_skinny_splits(0, M, N, K, 0) > 1, (M, N, K)
        a = t(bf(rng.standard_normal((M, K)).astype(np.float32)), torch.bfloat16)
        w = t(bf(rng.standard_normal((N, K)).astype(np.float32) * 0.1), torch.bfloat16)
        out = torch.empty(M, N, device=DEV)
        ops().gemm(out, a, w, kernel=kernel)
        cases.append((a, w, out, out.clone(), kernel))
        close(out, pm.linear(a.float().cpu().numpy(), w.float().cpu().numpy()), 1e-4, f"{M}x{N}x{K} {kernel}")
    differing = torch.zeros((), dtype=torch.int64, device=DEV)
    for _ in range(1000):
        for a, w, out, first, kernel in cases:
            ops().gemm(out, a, w, kernel=kernel)
            differing += (out != first).sum()
    assert int(differing) == 0


@pytest.mark.parametrize("M,N,K", [(130, 200, 256), (257, 97, 64), (1100, 1100, 640), (65, 70, 128), (2048, 896, 896), (2050, 2100, 192), (2048, 2176, 64), (1990, 890, 2048)])
def test_gemm_tiled_with_slabs_straight_into_lds(M, N, K):
    """K a multiple of 64 and not shared out: the forms of the tiled product whose slabs go from
    memory straight into a ring in LDS (rows past M and N are fetched from the last valid row, the
    chunks of a row lie permuted): small tiles with a ring of three, and big tiles with a ring of
    two where there are one to two of them per compute unit (the two shapes before the last), tiles
    of 128 x 64 with a ring of four where those fill the chip once and K is long (the last). Every epilogue
    they have, edges in both directions, one slab and many, and rows that are a strided view."""
    rng = np.random.default_rng(47)
    a, w = bf(rng.standard_normal((M, K)).astype(np.float32)), bf(rng.standard_normal((N, K)).astype(np.float32) * 0.1)
    b = rng.standard_normal(N).astype(np.float32)
    out = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    ops().gemm(out, t(a, torch.bfloat16), t(w, torch.bfloat16), t(b), kernel="tiled")
    close(out, pm.linear(a, w, b), BF16, "bf16 out")
    outf = torch.empty(M, N, device=DEV)
    ops().gemm(outf, t(a, torch.bfloat16), t(w, torch.bfloat16), kernel="tiled")
    close(outf, pm.linear(a, w), 1e-4, "f32 out")
    res = rng.standard_normal((M, N)).astype(np.float32)
    acc = t(res)
    ops().gemm(acc, t(a, torch.bfloat16), t(w, torch.bfloat16), add_to_out=True, kernel="tiled")
    close(acc, pm.add(res, pm.linear(a, w)), 1e-4, "residual")
    wide = torch.zeros(M, K + 72, device=DEV, dtype=torch.bfloat16)
    wide[:, 8:8 + K] = t(a, torch.bfloat16)
    ops().gemm(outf, wide[:, 8:8 + K], t(w, torch.bfloat16), kernel="tiled")
    close(outf, pm.linear(a, w), 1e-4, "rows that are a view")
    # a row's result does not depend on what else is in the batch, beyond the order of the additions (one row
    # alone makes few tiles, whose K may be shared out among blocks)
    one = torch.empty(1, N, device=DEV)
    ops().gemm(one, t(a[M - 1:], torch.bfloat16), t(w, torch.bfloat16), kernel="tiled")
    assert (one[0] - outf[M - 1]).abs().max().item() <= 2e-6 * outf[M - 1].abs().max().item()


@pytest.mark.parametrize("M,N,K", [(300, 400, 96), (256, 256, 32), (1, 5, 64), (513, 1030, 2080), (700, 130, 4096)])
def test_gemm_tiled_with_eight_waves_and_slabs_of_32(M, N, K):
    """The tiled product's form for many rows against a wide matrix (tiles of 256 x 256, eight waves, slabs of
    32 along K straight into a ring of four in LDS), asked for by name at sizes with edges in both directions,
    one slab and many, every epilogue it has, and rows that are a strided view; and the same bits as the tiled
    product's other forms give (one accumulator an output, ascending k, in all of them)."""
    rng = np.random.default_rng(48)
    a, w, w2 = (bf(rng.standard_normal((M, K)).astype(np.float32)), bf(rng.standard_normal((N, K)).astype(np.float32) * 0.1),
                bf(rng.standard_normal((N, K)).astype(np.float32) * 0.1))
    b = rng.standard_normal(N).astype(np.float32)
    ta, tw, tw2 = t(a, torch.bfloat16), t(w, torch.bfloat16), t(w2, torch.bfloat16)
    out = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    ops().gemm(out, ta, tw, t(b), kernel="wide")
    close(out, pm.linear(a, w, b), BF16, "bf16 out")
    outf = torch.empty(M, N, device=DEV)
    ops().gemm(outf, ta, tw, kernel="wide")
    close(outf, pm.linear(a, w), 1e-4, "f32 out")
    tiled = torch.empty(M, N, device=DEV)
    ops().gemm(tiled, ta, tw, kernel="tiled")
    if K < 2048:      # (with a long K and few tiles the tiled product shares K out over blocks: other sums)
        assert torch.equal(tiled, outf)
    res = rng.standard_normal((M, N)).astype(np.float32)
    acc = t(res)
    ops().gemm(acc, ta, tw, add_to_out=True, kernel="wide")
    close(acc, pm.add(res, pm.linear(a, w)), 1e-4, "residual")
    outs = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    ops().gemm_swiglu(outs, ta, tw, tw2, kernel="wide")
    close(outs, pm.swiglu(pm.linear(a, w), pm.linear(a, w2)), BF16, "swiglu")
    view = torch.zeros(M, K + 72, device=DEV, dtype=torch.bfloat16)
    view[:, 8:8 + K] = ta
    ops().gemm(outf, view[:, 8:8 + K], tw, kernel="wide")
    close(outf, pm.linear(a, w), 1e-4, "rows that are a view")
    with pytest.raises(AlofaError):
        ops().gemm(torch.empty(M, N, device=DEV), t(a[:, :K - 8].copy(), torch.bfloat16), t(w[:, :K - 8].copy(), torch.bfloat16), kernel="wide")      # K no multiple of 32


def test_the_tiled_product_takes_its_wide_form_where_the_rounds_are_full():
    """Many rows against a long K and tiles of 256 x 256 in nearly full rounds of the chip: the tiled product goes
    to the form above by itself; its sums are those of the forms it replaces (2,048 x 7,168 x 2,048: 224 tiles)."""
    rng = np.random.default_rng(49)
    M, N, K = 2048, 7168, 2048
    a = t(bf(rng.standard_normal((M, K)).astype(np.float32)), torch.bfloat16)
    w = t(bf(rng.standard_normal((N, K)).astype(np.float32) * 0.05), torch.bfloat16)
    by_rule, by_name = torch.empty(M, N, device=DEV, dtype=torch.bfloat16), torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    ops().gemm(by_rule, a, w, kernel="tiled")
    ops().gemm(by_name, a, w, kernel="wide")
    assert torch.equal(by_rule, by_name)
    rows = slice(1000, 1040)
    close(by_rule[rows], pm.linear(a[rows].float().cpu().numpy(), w.float().cpu().numpy()), BF16, "against the plain product")


@pytest.mark.parametrize("M,N,K", [(17, 1000, 128), (64, 4867, 896), (8, 18950, 2048), (33, 9000, 2112), (64, 14000, 2048), (5, 30, 64)])
def test_gate_and_up_of_one_tile_of_rows_in_blocks_dealt_out_evenly(M, N, K):
    """Up to 64 rows against gate and up matrices whose whole tiles are fewer than the compute units: the tiled
    product's blocks own as many columns as deal them out evenly (74 of a tile's 128 for 18,944 columns), the
    columns beyond are neither fetched nor stored. Odd column counts, every form the rule picks (tiles that hold
    32, 64 and 128 columns, short and long K), against the plain product."""
    rng = np.random.default_rng(50)
    a, w, w2 = (bf(rng.standard_normal((M, K)).astype(np.float32)), bf(rng.standard_normal((N, K)).astype(np.float32) * 0.05),
                bf(rng.standard_normal((N, K)).astype(np.float32) * 0.05))
    out = torch.full((M, N + 5), 7.0, device=DEV, dtype=torch.bfloat16)      # (a wider buffer: nothing is written beside the outputs)
    ops().gemm_swiglu(out[:, :N], t(a, torch.bfloat16), t(w, torch.bfloat16), t(w2, torch.bfloat16), kernel="tiled")
    close(out[:, :N], pm.swiglu(pm.linear(a, w), pm.linear(a, w2)), BF16, "gate/up")
    assert bool((out[:, N:] == 7.0).all())


def test_gemm_takes_a_strided_view():
    rng = np.random.default_rng(4)
    big = rng.standard_normal((6, 300)).astype(np.float32)
    w = rng.standard_normal((20, 100)).astype(np.float32)
    out = torch.empty(6, 20, device=DEV)
    ops().gemm(out, t(big)[:, 100:200], t(w), exact=True)
    close(out, pm.linear(big[:, 100:200], w), EXACT)


@pytest.mark.parametrize("M,N,K,kernel", with_kernels([(1, 176, 64), (37, 200, 240), (64, 130, 264), (130, 97, 80), (257, 176, 200), (300, 20000, 72)]))
def test_gemm_swiglu(M, N, K, kernel):
    rng = np.random.default_rng(5)
    a = rng.standard_normal((M, K)).astype(np.float32)
    wg, wu = rng.standard_normal((N, K)).astype(np.float32), rng.standard_normal((N, K)).astype(np.float32)
    out = torch.empty(M, N, device=DEV)
    ops().gemm_swiglu(out, t(a), t(wg), t(wu), exact=True)
    close(out, pm.swiglu(pm.linear(a, wg), pm.linear(a, wu)), EXACT, "exact")
    ab, gb, ub = bf(a), bf(wg * 0.2), bf(wu * 0.2)
    outb = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    ops().gemm_swiglu(outb, t(ab, torch.bfloat16), t(gb, torch.bfloat16), t(ub, torch.bfloat16), kernel=kernel)
    close(outb, pm.swiglu(pm.linear(ab, gb), pm.linear(ab, ub)), BF16, "bf16")
    g, u = rng.standard_normal((M, N)).astype(np.float32) * 8, rng.standard_normal((M, N)).astype(np.float32)
    g[0, 0] = -1e4                                                     # far negative gate: 0, not NaN
    sep = torch.empty(M, N, device=DEV)
    ops().swiglu(sep, t(g), t(u), exact=True)
    close(sep, pm.swiglu(g, u), EXACT, "unfused")


@pytest.mark.parametrize("heads,kv_heads,d,bs", [(6, 2, 48, 8), (3, 1, 32, 16), (4, 4, 128, 32)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rope_and_cache_write(heads, kv_heads, d, bs, dtype):
    rng = np.random.default_rng(6)
    T, n_blocks = 11, 7
    qkv = bf(rng.standard_normal((T, (heads + 2 * kv_heads) * d)).astype(np.float32))
    pos = rng.integers(0, 200, T)
    cos, sin = pm.rope_table(200, d, 1e4)
    slots = rng.permutation(n_blocks * bs)[:T]
    dev = t(qkv, dtype)
    kc = torch.full((n_blocks, kv_heads, bs, d), 7.0, device=DEV, dtype=dtype)
    vc = torch.full((n_blocks, kv_heads, d, bs), 7.0, device=DEV, dtype=dtype)       # values lie transposed: [channel][slot]
    ops().rope_kv_write(dev, t(cos[:, :d // 2]), t(sin[:, :d // 2]), t(pos.astype(np.int32), torch.int32), heads, kv_heads, d,
                        t(slots.astype(np.int64), torch.int64), kc, vc)
    rel = EXACT if dtype is torch.float32 else BF16
    q_ref = pm.rope_apply(qkv[:, :heads * d], cos, sin, pos, d)
    k_ref = pm.rope_apply(qkv[:, heads * d:(heads + kv_heads) * d], cos, sin, pos, d)
    close(dev[:, :heads * d], q_ref, rel, "q in place")
    kc_h, vc_h = kc.float().cpu().numpy(), vc.float().cpu().numpy().transpose(0, 1, 3, 2)
    written = np.zeros((n_blocks, bs), bool)
    for i, s in enumerate(slots):
        written[s // bs, s % bs] = True
        close(kc_h[s // bs, :, s % bs].reshape(-1), k_ref[i], rel, "k slot")
        assert np.array_equal(vc_h[s // bs, :, s % bs].reshape(-1), qkv[i, (heads + kv_heads) * d:])   # v is copied, not rotated
    assert (kc_h.transpose(0, 2, 1, 3)[~written] == 7.0).all() and (vc_h.transpose(0, 2, 1, 3)[~written] == 7.0).all()                               # other slots untouched


def paged_case(rng, lens, q_lens, heads, kv_heads, d, bs, dtype, scale_key=None):
    """Builds requests with their keys and values scattered over pages in a
    shuffled (not ascending) order, pages not in any table filled with NaN."""
    n_req = len(lens)
    blocks_per = [(L + bs - 1) // bs for L in lens]
    n_blocks = sum(blocks_per) + 3
    order = rng.permutation(n_blocks)
    kc = np.full((n_blocks, kv_heads, bs, d), np.nan, np.float32)
    vc = np.full((n_blocks, kv_heads, bs, d), np.nan, np.float32)
    table = np.full((n_req, max(blocks_per)), -1, np.int32)
    ks, vs, qs, pos, req = [], [], [], [], []
    used = 0
    for r, L in enumerate(lens):
        k = bf(rng.standard_normal((L, kv_heads * d)).astype(np.float32))
        v = bf(rng.standard_normal((L, kv_heads * d)).astype(np.float32))
        q = bf(rng.standard_normal((q_lens[r], heads * d)).astype(np.float32))
        if scale_key is not None:                  # one far key stands out for the last query of every head
            j = scale_key
            for h in range(heads):
                hk = h // (heads // kv_heads)
                q[-1, h * d:(h + 1) * d] = bf(6.0 * k[j, hk * d:(hk + 1) * d])
        table[r, :blocks_per[r]] = order[used:used + blocks_per[r]]
        used += blocks_per[r]
        for p in range(L):
            b = table[r, p // bs]
            kc[b, :, p % bs] = k[p].reshape(kv_heads, d)
            vc[b, :, p % bs] = v[p].reshape(kv_heads, d)
        ks.append(k), vs.append(v), qs.append(q)
        pos.extend(range(L - q_lens[r], L))
        req.extend([r] * q_lens[r])
    vc = vc.transpose(0, 1, 3, 2)      # the value cache is [block, kv_head, channel, slot]
    return dict(k=ks, v=vs, q=qs, kc=t(kc, dtype), vc=t(vc, dtype), table=t(table, torch.int32),
                pos=t(np.array(pos, np.int32), torch.int32), req=t(np.array(req, np.int32), torch.int32),
                qcat=t(np.concatenate(qs), dtype))


def test_exact_attention_on_the_reference_paged_vectors():
    """The reference's eleven paged-attention cases (tests/fixtures/paged/ there; its own test
    compares at one part in 1e5, tests/unit/test_paged_attention.mojo:66-70) as one batch of eleven
    requests through the float32 kernel: their gathered keys and values laid out in this engine's
    pages (whole pages of 16 slots in shuffled order, values transposed), the queries at the last
    positions; and its wrong-head-mapping control must not match."""
    from conftest import FIXTURES
    d_ = FIXTURES / "paged"
    floats = lambda f: np.array([float(x) for x in (d_ / f).read_text().split()], dtype=np.float32)      # noqa: E731
    cfg = dict(l.split("\t") for l in (d_ / "config.tsv").read_text().splitlines())
    bs, cols, H, Hkv, hd = (int(cfg[k]) for k in ("block_size", "kv_cols", "n_heads", "n_kv_heads", "head_dim"))
    cases = [l.split("\t") for l in (d_ / "cases.tsv").read_text().splitlines() if not l.startswith("#")]
    rng = np.random.default_rng(5)
    ks, vs, qs, wants = [], [], [], []
    for name, _s, _r, _o, q_len, _n, *_runs in cases:
        kv = floats(f"{name}.kv.tsv")
        L = kv.size // (2 * cols)
        ks.append(kv[:L * cols].reshape(L, cols)), vs.append(kv[L * cols:].reshape(L, cols))
        qs.append(floats(f"{name}.q.tsv").reshape(int(q_len), H * hd)), wants.append(floats(f"{name}.y.tsv").reshape(int(q_len), H * hd))
    per = [(k.shape[0] + bs - 1) // bs for k in ks]
    order = rng.permutation(sum(per) + 2)
    kc = np.full((sum(per) + 2, Hkv, bs, hd), np.nan, np.float32)
    vc = np.full_like(kc, np.nan)
    table = np.full((len(cases), max(per)), -1, np.int32)
    pos, req, used = [], [], 0
    for r, (k, v, q) in enumerate(zip(ks, vs, qs)):
        table[r, :per[r]] = order[used:used + per[r]]
        used += per[r]
        for p_ in range(k.shape[0]):
            kc[table[r, p_ // bs], :, p_ % bs] = k[p_].reshape(Hkv, hd)
            vc[table[r, p_ // bs], :, p_ % bs] = v[p_].reshape(Hkv, hd)
        pos.extend(range(k.shape[0] - q.shape[0], k.shape[0])), req.extend([r] * q.shape[0])
    out = torch.empty(len(pos), H * hd, device=DEV)
    ops().paged_attention(out, t(np.concatenate(qs)), t(kc), t(vc.transpose(0, 1, 3, 2)), t(table, torch.int32), t(np.array(req, np.int32), torch.int32),
                          t(np.array(pos, np.int32), torch.int32), H, Hkv, hd, None, float(np.float32(1) / np.sqrt(np.float32(hd))), True)
    want = np.concatenate(wants)
    close(out, want, 1e-5, "the reference's paged vectors")
    wrong = floats("expected_hmap.tsv").reshape(wants[0].shape)
    assert np.abs(out[:wrong.shape[0]].cpu().numpy() - wrong).max() > 1e-3


@pytest.mark.parametrize("heads,kv_heads,d,bs", [(6, 2, 48, 8), (8, 8, 16, 16), (5, 1, 80, 16), (4, 2, 128, 32), (2, 1, 256, 16), (14, 2, 64, 16)])
@pytest.mark.parametrize("dtype,exact", [(torch.float32, True), (torch.bfloat16, False)])
@pytest.mark.parametrize("window", [None, 21])
def test_paged_attention(heads, kv_heads, d, bs, dtype, exact, window):
    rng = np.random.default_rng(7)
    lens, q_lens = [37, 1, 130, 64], [37, 1, 5, 1]      # a whole prompt, a first token, a portion, a decode at a page's edge
    c = paged_case(rng, lens, q_lens, heads, kv_heads, d, bs, dtype)
    out = torch.empty(sum(q_lens), heads * d, device=DEV, dtype=dtype)
    scale = float(np.float32(1) / np.sqrt(np.float32(d)))
    ops().paged_attention(out, c["qcat"], c["kc"], c["vc"], c["table"], c["req"], c["pos"], heads, kv_heads, d, window, scale, exact)
    ref = np.concatenate([pm.attention(c["q"][r], c["k"][r], c["v"][r], heads, kv_heads, d, window) for r in range(4)])
    close(out, ref, 2e-6 if exact else BF16, "paged attention")


@pytest.mark.parametrize("heads,kv_heads,d,bs", [(6, 2, 48, 8), (8, 8, 16, 16), (5, 1, 80, 16), (4, 2, 128, 32), (2, 1, 256, 16), (14, 2, 64, 16), (18, 2, 32, 64), (20, 1, 32, 16)])
@pytest.mark.parametrize("window", [None, 21, 300])
@pytest.mark.parametrize("bucket", [700, 2048, 8192])
def test_decode_attention(heads, kv_heads, d, bs, window, bucket):
    """The kernel for few query tokens per request: single tokens and short
    portions, contexts from one key to many pages, groups of 1 to 9 heads per
    key head, head sizes whose lanes-per-key is no power of two. ``bucket`` is the
    context bound the launch is shaped for: the waves of one block share the keys
    out, and for the larger bounds several blocks do, whose states a second kernel combines."""
    rng = np.random.default_rng(17)
    lens, q_lens = [1, 37, 700, 64, 333], [1, 2, 1, 4, 3]
    c = paged_case(rng, lens, q_lens, heads, kv_heads, d, bs, torch.bfloat16)
    out = torch.empty(sum(q_lens), heads * d, device=DEV, dtype=torch.bfloat16)
    scale = float(np.float32(1) / np.sqrt(np.float32(d)))
    o = ops()
    scratch = torch.empty(max(1, o.decode_scratch_floats(sum(q_lens), heads, kv_heads, d, bucket, window)), device=DEV)
    o.paged_attention(out, c["qcat"], c["kc"], c["vc"], c["table"], c["req"], c["pos"], heads, kv_heads, d, window, scale, False,
                      max_q_len=4, max_context=bucket, scratch=scratch)
    ref = np.concatenate([pm.attention(c["q"][r], c["k"][r], c["v"][r], heads, kv_heads, d, window) for r in range(5)])
    close(out, ref, BF16, "decode attention")
    if (heads, d, window) == (14, 64, None):
        assert o.decode_splits(sum(q_lens), heads, kv_heads, d, bucket) == {700: 4, 2048: 8, 8192: 11}[bucket]   # several parts are really in play (256 // 22 blocks)
    one = torch.empty(1, heads * d, device=DEV, dtype=torch.bfloat16)        # one token that sees one key
    o.paged_attention(one, c["qcat"][:1], c["kc"], c["vc"], c["table"], c["req"][:1], c["pos"][:1], heads, kv_heads, d, window, scale, False,
                      max_q_len=1, max_context=1)
    close(one, ref[:1], BF16, "decode attention, first token")
    if o.decode_scratch_floats(sum(q_lens), heads, kv_heads, d, bucket, window):
        from alofa_amd.errors import AlofaError
        with pytest.raises(AlofaError):                                          # needed scratch is demanded, not allocated behind the back
            o.paged_attention(out, c["qcat"], c["kc"], c["vc"], c["table"], c["req"], c["pos"], heads, kv_heads, d, window, scale, False,
                              max_q_len=4, max_context=bucket)
    # both ways in which parts meet, whatever the launch would choose: the last block combines them, or a second kernel does
    for parts in (2, 4, 7, 8, 13):
        for hand_over in (True, False):
            again = torch.zeros_like(out)
            o.attention_decode(again, c["qcat"], c["kc"], c["vc"], c["table"], c["req"], c["pos"], heads, kv_heads, d, window, scale, bucket,
                               torch.empty(sum(q_lens) * heads * parts * (d + 2), device=DEV), n_splits=parts, hand_over=hand_over)
            close(again, ref, BF16, f"decode attention, {parts} parts, hand-over {hand_over}")


@pytest.mark.parametrize("heads,kv_heads,d,bs", [(14, 2, 64, 16), (8, 2, 128, 32), (20, 1, 64, 8), (3, 3, 256, 16)])
@pytest.mark.parametrize("window", [None, 21])
@pytest.mark.parametrize("bucket", [700, 8192])
def test_decode_attention_that_rotates_and_writes_the_new_token(heads, kv_heads, d, bs, window, bucket):
    """One new token per request, handed over as the fused projection's row [queries | keys | values]
    before rotation: the kernel rotates queries and the new key, attends over the cache and the new
    token, and writes the new key and value to the token's slot (which holds NaN before)."""
    rng = np.random.default_rng(19)
    lens, n = [1, 37, 700, 64, 333, 16, 17], 7
    c = paged_case(rng, lens, [1] * n, heads, kv_heads, d, bs, torch.bfloat16)
    cos, sin = pm.rope_table(max(lens), d, 1e4)
    o = ops()
    assert o.can_fuse_rope_into_decode(d)
    qkv = np.zeros((n, (heads + 2 * kv_heads) * d), np.float32)
    kc, vc = c["kc"].clone(), c["vc"].clone()
    slots, refs = [], []
    table = c["table"].cpu().numpy()
    for r, L in enumerate(lens):
        q_raw = bf(rng.standard_normal((1, heads * d)).astype(np.float32))
        k_raw = bf(rng.standard_normal((1, kv_heads * d)).astype(np.float32))
        pos = np.array([L - 1])
        q_rot = bf(pm.rope_apply(q_raw, cos, sin, pos, d).astype(np.float32))
        k_rot = bf(pm.rope_apply(k_raw, cos, sin, pos, d).astype(np.float32))
        k = c["k"][r].copy()
        k[L - 1] = k_rot[0]                          # what the cache must hold for the new token afterwards
        qkv[r] = np.concatenate([q_raw[0], k_raw[0], c["v"][r][L - 1]])
        slot = int(table[r, (L - 1) // bs]) * bs + (L - 1) % bs
        slots.append(slot)
        kc[slot // bs, :, slot % bs] = float("nan")                          # not written yet
        vc[slot // bs, :, :, slot % bs] = float("nan")
        refs.append((pm.attention(q_rot, k, c["v"][r], heads, kv_heads, d, window), k_rot[0], c["v"][r][L - 1]))
    out = torch.empty(n, heads * d, device=DEV, dtype=torch.bfloat16)
    scale = float(np.float32(1) / np.sqrt(np.float32(d)))
    scratch = torch.empty(max(1, o.decode_scratch_floats(n, heads, kv_heads, d, bucket, window)), device=DEV)
    o.attention_decode(out, t(qkv, torch.bfloat16), kc, vc, c["table"], c["req"], c["pos"], heads, kv_heads, d, window, scale, bucket, scratch,
                       rope=(t(cos[:, :d // 2]), t(sin[:, :d // 2]), t(np.array(slots, np.int64), torch.int64)))
    close(out, np.concatenate([a for a, _, _ in refs]), BF16, "attention with the new token from registers")
    kc_h, vc_h = kc.float().cpu().numpy(), vc.float().cpu().numpy()
    for r, slot in enumerate(slots):
        close(kc_h[slot // bs, :, slot % bs].reshape(-1), refs[r][1], BF16, "new key in its slot")
        assert np.array_equal(vc_h[slot // bs, :, :, slot % bs].reshape(-1), refs[r][2]), "new value in its slot"
    # one token per request, in table order: the request indices may be left out, and nothing changes
    again = torch.empty_like(out)
    o.attention_decode(again, t(qkv, torch.bfloat16), kc, vc, c["table"], None, c["pos"], heads, kv_heads, d, window, scale, bucket, scratch,
                       rope=(t(cos[:, :d // 2]), t(sin[:, :d // 2]), t(np.array(slots, np.int64), torch.int64)))
    assert torch.equal(again, out)
    with pytest.raises(AlofaError):
        o.attention_decode(again, t(qkv, torch.bfloat16), kc, vc, c["table"][:n - 1], None, c["pos"], heads, kv_heads, d, window, scale, bucket, scratch)


@pytest.mark.parametrize("heads,kv_heads,d", [(5, 1, 80), (2, 2, 96), (3, 1, 64)])
def test_decode_attention_with_many_splits(heads, kv_heads, d):
    """One token over 5,000 keys, the launch shaped for a far longer context: the keys are shared out
    among 64 parts, and all of them count (head sizes between 64 and 128 combine channels 64.. in a
    second round of the lanes)."""
    rng = np.random.default_rng(18)
    lens, q_lens = [5000, 3000], [1, 2]
    c = paged_case(rng, lens, q_lens, heads, kv_heads, d, 16, torch.bfloat16)
    out = torch.empty(sum(q_lens), heads * d, device=DEV, dtype=torch.bfloat16)
    scale = float(np.float32(1) / np.sqrt(np.float32(d)))
    o = ops()
    assert o.decode_splits(sum(q_lens), heads, kv_heads, d, 65536) >= 32
    scratch = torch.empty(o.decode_scratch_floats(sum(q_lens), heads, kv_heads, d, 65536, None), device=DEV)
    o.paged_attention(out, c["qcat"], c["kc"], c["vc"], c["table"], c["req"], c["pos"], heads, kv_heads, d, None, scale, False,
                      max_q_len=2, max_context=65536, scratch=scratch)
    ref = np.concatenate([pm.attention(c["q"][r], c["k"][r], c["v"][r], heads, kv_heads, d, None) for r in range(2)])
    # random keys give almost even weights, so the result is small: compare at its own scale
    err = np.abs(out.float().cpu().numpy() - ref).max()
    assert err <= 1e-2 * np.abs(ref).max(), f"{err} vs {np.abs(ref).max()}"


def long_case(rng, lens, q_lens, heads, kv_heads, d, bs, peak=1.2, holes=None, far=None):
    """Requests over long contexts, built without a loop per position: request r sees the first ``lens[r]`` of one
    shared run of random keys and values, laid out on pages of its own in shuffled order; its queries are the last
    ``q_lens[r]`` positions. Every last query leans towards one key near the start of its context (3 + 5 r): with
    ``peak`` 1.2 that key carries about a fifth of the weight among tens of thousands, so both a dropped far key
    and a wrong sum over the many show at the result's own scale (``far[r]``: another place for it). ``holes[r]``: so many leading pages are missing
    from the table (-1), as behind a window that has passed them. Pages in no table hold NaN."""
    L = max(lens)
    k = bf(rng.standard_normal((L, kv_heads * d)).astype(np.float32))
    v = bf(rng.standard_normal((L, kv_heads * d)).astype(np.float32))
    per = [(n + bs - 1) // bs for n in lens]
    n_blocks = sum(per) + 3
    order = rng.permutation(n_blocks)
    kc = torch.full((n_blocks, kv_heads, bs, d), float("nan"), dtype=torch.bfloat16)
    vc = torch.full((n_blocks, kv_heads, bs, d), float("nan"), dtype=torch.bfloat16)
    k_t, v_t = torch.from_numpy(k).to(torch.bfloat16).view(L, kv_heads, d), torch.from_numpy(v).to(torch.bfloat16).view(L, kv_heads, d)
    table = np.full((len(lens), max(per)), -1, np.int32)
    qs, pos, req, used = [], [], [], 0
    for r, n in enumerate(lens):
        table[r, :per[r]] = order[used:used + per[r]]
        used += per[r]
        at = np.arange(n)
        first = (holes[r] if holes else 0) * bs
        pages, places = torch.from_numpy(table[r, at[first:] // bs].astype(np.int64)), torch.from_numpy(at[first:] % bs)
        kc[pages, :, places] = k_t[first:n]
        vc[pages, :, places] = v_t[first:n]
        if holes:
            table[r, :holes[r]] = -1
        q = bf(rng.standard_normal((q_lens[r], heads * d)).astype(np.float32))
        j = far[r] if far else 3 + 5 * r
        for h in range(heads):
            hk = h // (heads // kv_heads)
            q[-1, h * d:(h + 1) * d] = bf(peak * k[j, hk * d:(hk + 1) * d])
        qs.append(q)
        pos.extend(range(n - q_lens[r], n))
        req.extend([r] * q_lens[r])
    return dict(k=k, v=v, q=qs, kc=kc.to(DEV), vc=vc.transpose(2, 3).contiguous().to(DEV), table=t(table, torch.int32),
                pos=t(np.array(pos, np.int32), torch.int32), req=t(np.array(req, np.int32), torch.int32),
                qcat=t(np.concatenate(qs), torch.bfloat16), lens=lens)


def long_reference(c, r, heads, kv_heads, d, window=None, rows=None):
    """The plain attention of request r's queries (the last ``rows`` of them) over its context."""
    n = c["lens"][r]
    q = c["q"][r] if rows is None else c["q"][r][-rows:]
    return pm.attention(q, c["k"][:n], c["v"][:n], heads, kv_heads, d, window)


def close_at_own_scale(got, ref, what):
    """Attention over tens of thousands of random keys is small: compared at the result's own scale, within the
    eight bits of a bfloat16 output and weights."""
    got = got.detach().float().cpu().numpy() if isinstance(got, torch.Tensor) else got
    err, scale = np.abs(got.astype(np.float64) - ref).max(), np.abs(ref).max()
    assert np.isfinite(got).all() and err <= 1.5e-2 * scale, f"{what}: {err:.3e} > 1.5e-2 x {scale:.3e}"


@pytest.mark.parametrize("batch", [1, 8])
@pytest.mark.parametrize("context", [8192, 16384, 32768])
@pytest.mark.parametrize("heads,kv_heads,d", [(14, 2, 64), (28, 4, 128)])
def test_decode_attention_at_the_contexts_that_are_timed(heads, kv_heads, d, context, batch):
    """One token per request over 8,192 to 32,768 real keys (every part of the context holds data, and a far key
    carries weight): the parts the launch rule picks at that context, merged by the second kernel or handed over to
    the last block, eight parts handed over, and the form that rotates and writes the new token itself."""
    rng = np.random.default_rng(61)
    o = ops()
    lens = [context - 37 * r for r in range(batch)]
    c = long_case(rng, lens, [1] * batch, heads, kv_heads, d, 16)
    scale = float(np.float32(1) / np.sqrt(np.float32(d)))
    ref = np.concatenate([long_reference(c, r, heads, kv_heads, d) for r in range(batch)])
    assert np.abs(ref).max() > 0.15                                     # the far key counts
    picked = o.decode_splits(batch, heads, kv_heads, d, context)
    assert picked >= 8
    out = torch.zeros(batch, heads * d, device=DEV, dtype=torch.bfloat16)
    scratch = torch.empty(max(1, o.decode_scratch_floats(batch, heads, kv_heads, d, context, None)), device=DEV)
    o.paged_attention(out, c["qcat"], c["kc"], c["vc"], c["table"], c["req"], c["pos"], heads, kv_heads, d, None, scale, False,
                      max_q_len=1, max_context=context, scratch=scratch)
    close_at_own_scale(out, ref, f"{picked} parts, as the rule picks")
    big = torch.empty(batch * heads * 64 * (d + 2), device=DEV)
    can_hand_over = o.decode_hand_over(batch, heads, kv_heads, d, 8)
    assert can_hand_over or batch > 1
    for parts, hand_over in ((picked, False), (8, True), (8, False), (64 if batch == 1 else 32, False)):
        if hand_over and not can_hand_over:
            continue
        out.zero_()
        o.attention_decode(out, c["qcat"], c["kc"], c["vc"], c["table"], c["req"], c["pos"], heads, kv_heads, d, None, scale, context, big,
                           n_splits=parts, hand_over=hand_over)
        close_at_own_scale(out, ref, f"{parts} parts, hand-over {hand_over}")
    # the new token arrives as the fused projection's row, not yet rotated; its slot holds NaN before
    cos, sin = pm.rope_table(context, d, 1e6)
    qkv = np.zeros((batch, (heads + 2 * kv_heads) * d), np.float32)
    slots, table = [], c["table"].cpu().numpy()
    kc, vc = c["kc"].clone(), c["vc"].clone()
    refs = []
    for r, n in enumerate(lens):
        q_raw, k_raw = c["q"][r], bf(rng.standard_normal((1, kv_heads * d)).astype(np.float32))
        at = np.array([n - 1])
        q_rot, k_rot = bf(pm.rope_apply(q_raw, cos, sin, at, d)), bf(pm.rope_apply(k_raw, cos, sin, at, d))
        k = c["k"][:n].copy()
        k[n - 1] = k_rot[0]
        qkv[r] = np.concatenate([q_raw[0], k_raw[0], c["v"][n - 1]])
        slot = int(table[r, (n - 1) // 16]) * 16 + (n - 1) % 16
        slots.append(slot)
        kc[slot // 16, :, slot % 16] = float("nan")
        vc[slot // 16, :, :, slot % 16] = float("nan")
        refs.append(pm.attention(q_rot, k, c["v"][:n], heads, kv_heads, d))
    rope = (t(cos[:, :d // 2]), t(sin[:, :d // 2]), t(np.array(slots, np.int64), torch.int64))
    for parts, hand_over in ((picked, False), (8, True)):
        if hand_over and not can_hand_over:
            continue
        kc2, vc2 = kc.clone(), vc.clone()
        out.zero_()
        o.attention_decode(out, t(qkv, torch.bfloat16), kc2, vc2, c["table"], None, c["pos"], heads, kv_heads, d, None, scale, context, big,
                           rope=rope, n_splits=parts, hand_over=hand_over)
        close_at_own_scale(out, np.concatenate(refs), f"rotating form, {parts} parts, hand-over {hand_over}")
        for slot in slots:
            assert torch.isfinite(kc2[slot // 16, :, slot % 16].float()).all() and torch.isfinite(vc2[slot // 16, :, :, slot % 16].float()).all()


@pytest.mark.parametrize("heads,kv_heads,d,shares", [(14, 2, 64, (0, 7)), (40, 8, 128, (0,)), (16, 2, 64, (0, 8))])
@pytest.mark.parametrize("window", [None, 3000])
def test_prefill_attention_of_portions_deep_in_a_context(heads, kv_heads, d, shares, window):
    """A portion of 64 and one of 200 rows that start at position 16,000 (the portions of a long prompt's later
    steps): every form the kernel has for these heads (a block per head with 16 rows a wave, and with 32 rows and
    tiles of 32 keys at head size 128; the heads of a group sharing their tiles, with 16 and 32 rows a wave), the
    last rows against the plain attention. With a window, the pages that the window has passed are gone from the
    table (-1), as the cache manager leaves them."""
    rng = np.random.default_rng(67)
    o = ops()
    start, bs = 16000, 16
    lens, q_lens = [start + 64, start + 200], [64, 200]
    holes = [max(0, (n - q - window + 1)) // bs for n, q in zip(lens, q_lens)] if window else None
    far = [n - window + 2 + 5 * r for r, n in enumerate(lens)] if window else None      # just inside the last row's window
    c = long_case(rng, lens, q_lens, heads, kv_heads, d, bs, holes=holes, far=far)
    scale = float(np.float32(1) / np.sqrt(np.float32(d)))
    checked = 24                                                       # rows of every request that the plain side computes
    ref = [long_reference(c, r, heads, kv_heads, d, window, rows=checked) for r in range(2)]
    assert min(np.abs(x[-1]).max() for x in ref) > 0.15                 # the far key counts in the last rows
    tiles, row = [], 0
    for r, (L, n) in enumerate(zip(lens, q_lens)):
        tiles += [(r, row + q0, min(64, n - q0), L - n + q0) for q0 in range(0, n, 64)]
        row += n
    out = torch.zeros(sum(q_lens), heads * d, device=DEV, dtype=torch.bfloat16)
    forms = [(share, rows) for share in shares for rows in ((16, 32) if (share and d in (32, 64, 96)) or (not share and d == 128) else (16,))]
    assert len(forms) >= 2
    for share, rows in forms:
        for name, blocks in (("paired", o.pair_tiles(tiles, window)), ("single", o.pair_tiles(tiles, window, 1))):
            out.zero_()
            o.attention_prefill(out, c["qcat"], c["kc"], c["vc"], c["table"], t(np.array(blocks, np.int32), torch.int32), heads, kv_heads, d, window, scale,
                                share=share, rows=rows)
            got = out.float().cpu().numpy()
            assert np.isfinite(got).all()
            close_at_own_scale(got[64 - checked:64], ref[0], f"64 rows at {start}, {name}, {share} share, {rows} rows a wave")
            close_at_own_scale(got[264 - checked:264], ref[1], f"200 rows at {start}, {name}, {share} share, {rows} rows a wave")


@pytest.mark.parametrize("heads,kv_heads,d,bs", [(6, 2, 48, 8), (8, 8, 16, 16), (5, 1, 96, 16), (4, 2, 128, 32), (2, 1, 256, 16), (14, 2, 64, 16), (3, 1, 32, 64),
                                                 (22, 2, 32, 16), (6, 1, 256, 16), (28, 4, 128, 16), (7, 1, 16, 8), (16, 2, 64, 16), (6, 1, 96, 16)])
@pytest.mark.parametrize("window", [None, 21, 300])
def test_prefill_attention(heads, kv_heads, d, bs, window):
    """The tiled kernel for portions of prompts: whole prompts, portions deep in
    a context, runs of exactly 64 and 65 rows, several tiles per request. A block serves 64 rows of
    one head, or, in launches with many blocks and six or more query heads per key head (head sizes up
    to 128), 16 rows of the heads of a group, which share the staged tiles (groups of six to eight in
    teams of as many waves, eleven in chunks of six and five), or 32 rows of them where the head size is 32,
    64 or 96; at head size 128 a block of one head also comes with 32 rows a wave and tiles of 32 keys: every
    form is run where it exists."""
    rng = np.random.default_rng(23)
    lens, q_lens = [37, 130, 700, 64, 65, 200], [37, 5, 100, 64, 65, 200]
    c = paged_case(rng, lens, q_lens, heads, kv_heads, d, bs, torch.bfloat16)
    tiles, row = [], 0
    for r, (L, n) in enumerate(zip(lens, q_lens)):
        tiles += [(r, row + q0, min(64, n - q0), L - n + q0) for q0 in range(0, n, 64)]
        row += n
    out = torch.zeros(sum(q_lens), heads * d, device=DEV, dtype=torch.bfloat16)
    scale = float(np.float32(1) / np.sqrt(np.float32(d)))
    ref = np.concatenate([pm.attention(c["q"][r], c["k"][r], c["v"][r], heads, kv_heads, d, window) for r in range(len(lens))])
    # two runs per block (many blocks) and a block per run (fewer blocks than compute units)
    paired, single = ops().pair_tiles(tiles, window), ops().pair_tiles(tiles, window, 1)
    assert sorted(tuple(r) for b in paired for r in b if r[2]) == sorted(tiles) and len(paired) == (len(tiles) + 1) // 2
    assert [tuple(b[0]) for b in single] == tiles and all(b[1][2] == 0 for b in single)
    assert len(ops().pair_tiles(tiles * 40, window, heads)) == len(tiles) * 20
    # the kernel's own choice for a launch of few runs and of very many
    group = heads // kv_heads
    wide = ops().prefill_share(heads, kv_heads, d, 1 << 20)
    assert ops().prefill_share(heads, kv_heads, d, 1) == 0
    assert wide == {1: 0, 2: 0, 3: 0, 5: 0, 6: 6 if d <= 128 else 0, 7: 7, 8: 8, 11: 6}[group]
    rows32 = bool(wide) and d in (32, 64, 96)
    assert ops().prefill_rows(heads, kv_heads, d, wide, 1 << 20) == (32 if rows32 or (d == 128 and not wide) else 16)
    assert ops().prefill_rows(heads, kv_heads, d, 0, 1 << 20) == (32 if d == 128 else 16) and ops().prefill_rows(heads, kv_heads, d, 0, 1) == 16
    if rows32:     # blocks of 32 rows from one and a half per compute unit on
        per_run, cus = kv_heads * -(-group // wide) * 2, ops().compute_units()
        assert ops().prefill_rows(heads, kv_heads, d, wide, -(-3 * cus // (2 * per_run))) == 32
        assert ops().prefill_rows(heads, kv_heads, d, wide, -(-3 * cus // (2 * per_run)) - 1) == 16
    assert ops().prefill_blocks_per_run(heads, kv_heads, wide) == (kv_heads * -(-group // wide) * 4 if wide else heads)
    assert ops().prefill_blocks_per_run(heads, kv_heads, wide, 32) == (kv_heads * -(-group // wide) * 2 if wide else heads)
    for share, rows in [(0, 16)] + ([(0, 32)] if d == 128 else []) + ([(wide, 16)] if wide else []) + ([(wide, 32)] if rows32 else []):
        for name, blocks in (("paired", paired), ("single", single)):
            out.zero_()
            ops().attention_prefill(out, c["qcat"], c["kc"], c["vc"], c["table"], t(np.array(blocks, np.int32), torch.int32), heads, kv_heads, d, window, scale,
                                    share=share, rows=rows)
            close(out, ref, BF16, f"prefill attention, {name}, {share} heads share, {rows} rows a wave")
    if d != 128 or wide:
        with pytest.raises(Exception, match="rows a wave"):
            ops().attention_prefill(out, c["qcat"], c["kc"], c["vc"], c["table"], t(np.array(single, np.int32), torch.int32), heads, kv_heads, d, window, scale,
                                    share=wide if d == 128 else 0, rows=32)
    with pytest.raises(Exception, match="cannot share"):
        ops().attention_prefill(out, c["qcat"], c["kc"], c["vc"], c["table"], t(np.array(single, np.int32), torch.int32), heads, kv_heads, d, window, scale,
                                share=5)


def test_prefill_attention_far_key():
    rng = np.random.default_rng(29)
    heads, kv_heads, d, bs, L, far = 6, 2, 64, 16, 700, 3
    c = paged_case(rng, [L], [40], heads, kv_heads, d, bs, torch.bfloat16, scale_key=far)
    out = torch.zeros(40, heads * d, device=DEV, dtype=torch.bfloat16)
    scale = float(np.float32(1) / np.sqrt(np.float32(d)))
    for window in (None, L - far, L - far - 1):
        ops().attention_prefill(out, c["qcat"], c["kc"], c["vc"], c["table"], t(np.array([[[0, 0, 40, L - 40], [0, 0, 0, 0]]], np.int32), torch.int32),
                                heads, kv_heads, d, window, scale)
        close(out, pm.attention(c["q"][0], c["k"][0], c["v"][0], heads, kv_heads, d, window), BF16, f"far key, window {window}")


@pytest.mark.parametrize("dtype,exact", [(torch.float32, True), (torch.bfloat16, False)])
def test_attention_far_key_and_window_edge(dtype, exact):
    """One far key among hundreds carries the weight: dropping it, or any page of
    the table, shows. With a window the same key is cut off exactly at the edge."""
    rng = np.random.default_rng(8)
    heads, kv_heads, d, bs, L, far = 6, 2, 64, 16, 700, 3
    c = paged_case(rng, [L], [1], heads, kv_heads, d, bs, dtype, scale_key=far)
    scale = float(np.float32(1) / np.sqrt(np.float32(d)))
    out = torch.empty(1, heads * d, device=DEV, dtype=dtype)
    ops().paged_attention(out, c["qcat"], c["kc"], c["vc"], c["table"], c["req"], c["pos"], heads, kv_heads, d, None, scale, exact)
    ref = pm.attention(c["q"][0], c["k"][0], c["v"][0], heads, kv_heads, d)
    close(out, ref, 2e-6 if exact else BF16, "far key")
    v_far = np.concatenate([c["v"][0][far, (h // 3) * d:(h // 3 + 1) * d] for h in range(heads)])
    assert np.abs(ref[0] - v_far).max() < 1e-3                          # the far key really decides the output
    for window, sees in ((L - far, True), (L - far - 1, False)):         # the window's edge, to the key
        ops().paged_attention(out, c["qcat"], c["kc"], c["vc"], c["table"], c["req"], c["pos"], heads, kv_heads, d, window, scale, exact,
                              max_q_len=None if exact else 1, max_context=L, scratch=torch.empty(1 << 16, device=DEV))
        refw = pm.attention(c["q"][0], c["k"][0], c["v"][0], heads, kv_heads, d, window)
        close(out, refw, 2e-6 if exact else BF16, f"window {window}")
        assert (np.abs(refw[0] - v_far).max() < 1e-3) == sees


def test_argmax_and_sample():
    rng = np.random.default_rng(9)
    vocab = 1537
    logits = rng.standard_normal((5, vocab)).astype(np.float32)
    logits[1, [40, 900, 7]] = 9.0          # ties: the lowest index wins
    logits[2, :] = -3.0                    # all equal
    out = torch.empty(5, dtype=torch.int32, device=DEV)
    ops().argmax(out, t(logits))
    assert out.tolist() == [pm.argmax(r) for r in logits] and out[1].item() == 7 and out[2].item() == 0
    big = rng.standard_normal((3, 151936)).astype(np.float32)       # long rows take the two-stage search
    big[0, [150000, 2400, 77000]] = 11.0
    big[1, :] = 2.0
    big[2, 151935] = 12.0
    outb = torch.empty(3, dtype=torch.int32, device=DEV)
    ops().argmax(outb, t(big))
    assert outb.tolist() == [2400, 0, 151935]
    rows = np.repeat(logits[:1], 64, axis=0)
    temps = np.full(64, 0.8)
    us = np.array([ps.SplitMix64(3).next_uniform() for _ in range(1)] + list(rng.random(61)) + [0.0, 0.9999999999999999])
    picks = torch.empty(64, dtype=torch.int32, device=DEV)
    ops().sample(picks, t(rows), t(temps, torch.float64), t(us, torch.float64))
    _, p = ps.distribution(logits[0], temperature=0.8)
    assert picks.tolist() == [ps.pick_from(p, u) for u in us]
    # a low temperature converges to the greedy choice
    ops().sample(picks, t(rows), t(np.full(64, 1e-4), torch.float64), t(np.clip(us, 0.01, 0.99), torch.float64))
    assert set(picks.tolist()) == {int(np.argmax(logits[0]))}


def test_kernels_refuse_what_they_cannot_take():
    from alofa_amd.errors import AlofaError
    o = ops()
    with pytest.raises(AlofaError):
        o.gemm(torch.empty(2, 3, device=DEV), torch.empty(2, 4, device=DEV), torch.empty(3, 5, device=DEV))
    with pytest.raises(AlofaError):
        o.gemm(torch.empty(2, 3), torch.empty(2, 4), torch.empty(3, 4))                  # not on the GPU
    with pytest.raises(AlofaError):
        o.rmsnorm(torch.empty(2, 8, device=DEV, dtype=torch.bfloat16), torch.empty(2, 8, device=DEV), torch.empty(8, device=DEV), 1e-6, True)
    with pytest.raises(AlofaError):
        o.argmax(torch.empty(2, dtype=torch.int32, device=DEV), torch.empty(3, 8, device=DEV))
    # a product that adds to the residual stream takes no bias, in either dtype (no kernel would add it)
    for dt in (torch.float32, torch.bfloat16):
        with pytest.raises(AlofaError) as e:
            o.gemm(torch.zeros(2, 8, device=DEV), torch.zeros(2, 16, device=DEV, dtype=dt), torch.zeros(8, 16, device=DEV, dtype=dt),
                   torch.zeros(8, device=DEV), add_to_out=True, exact=dt is torch.float32)
        assert e.value.name == "unsupported"


@pytest.mark.parametrize("M,N,K", [(1, 32768, 72), (8, 40011, 200), (37, 33000, 896), (64, 151936, 64)])
def test_product_with_the_argmax_on_it(M, N, K):
    """The vocabulary product that leaves, instead of its outputs, the best column per row: the
    same choice as the product followed by the argmax kernels, value for value, also where whole
    rows are full of equal values (small integers as operands: the lowest index must win, within a
    wave's two tiles, between waves, between blocks), past the matrix's end (N no multiple of 128),
    and with the choice going to a token store."""
    o = ops()
    rng = np.random.default_rng(53)
    for kind in ("integers", "normal"):
        if kind == "integers":
            a = rng.integers(-1, 2, (M, K)).astype(np.float32)
            w = rng.integers(-1, 2, (N, K)).astype(np.float32)
        else:
            a, w = bf(rng.standard_normal((M, K)).astype(np.float32)), bf(rng.standard_normal((N, K)).astype(np.float32) * 0.1)
        at, wt = t(a, torch.bfloat16), t(w, torch.bfloat16)
        assert o.can_gemm_argmax(M, wt)
        logits = torch.empty(M, N, device=DEV)
        o.gemm(logits, at, wt)
        two_steps = torch.empty(M, dtype=torch.int32, device=DEV)
        o.argmax(two_steps, logits)
        fused = torch.full((M,), -1, dtype=torch.int32, device=DEV)
        o.gemm_argmax(fused, at, wt)
        assert torch.equal(fused, two_steps), kind
        ref = pm.linear(a, w)
        assert np.array_equal(ref[np.arange(M), fused.cpu().numpy()], ref.max(1)) or kind == "normal"
        if kind == "integers":     # exact sums: the plain product's first maximum is the answer
            assert np.array_equal(fused.cpu().numpy(), ref.argmax(1))
    store = torch.full((100,), -7, dtype=torch.int32, device=DEV)
    index = t(rng.permutation(100)[:M].astype(np.int32), torch.int32)
    again = torch.empty(M, dtype=torch.int32, device=DEV)
    o.gemm_argmax(again, at, wt, store=store, store_index=index)
    assert torch.equal(again, fused) and torch.equal(store[index.long()], fused) and int((store != -7).sum()) == M
    with pytest.raises(AlofaError):
        o.gemm_argmax(torch.empty(65, dtype=torch.int32, device=DEV), torch.zeros(65, K, device=DEV, dtype=torch.bfloat16), wt)


def test_product_kernel_choice():
    """The choice between the two bfloat16 products: few rows and small weights stream, many
    rows or big weights are tiled; a kernel that cannot take the rows is an error, not a guess."""
    o = ops()
    assert o.few_rows_kernel(1, 151936, 896) == "tiled" and o.few_rows_kernel(1, 2 * 18944, 3584, swiglu=True) == "rows"
    assert o.few_rows_kernel(4, 4608, 3584) == "rows" and o.few_rows_kernel(2, 3584, 18944) == "rows" and o.few_rows_kernel(4, 5120, 13824) == "rows" and o.few_rows_kernel(8, 3584, 18944) == "tiled"
    assert o.few_rows_kernel(64, 2 * 4864, 896, swiglu=True) == "tiled" and o.few_rows_kernel(16, 2 * 4864, 896, swiglu=True) == "stream"
    assert o.few_rows_kernel(64, 896, 4864) == "stream" and o.few_rows_kernel(32, 3584, 3584) == "tiled"
    assert o.few_rows_kernel(65, 8, 8) == "tiled"
    a, w = torch.zeros(70, 64, device=DEV, dtype=torch.bfloat16), torch.zeros(16, 64, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(AlofaError):
        o.gemm(torch.empty(70, 16, device=DEV), a, w, kernel="stream")


@pytest.mark.parametrize("M,N,K", [(17, 4000, 128), (40, 3990, 192), (64, 1000, 896), (64, 330, 2112), (190, 1000, 64), (300, 4000, 128), (520, 4000, 192), (1030, 4000, 64), (130, 97, 3584)])
def test_gate_up_tiled_with_slabs_straight_into_lds(M, N, K):
    """Gate/up with K a multiple of 64 through the tiled kernel: tiles of 64 rows with a ring of four or three slabs
    (of 32 outputs where the tiles are few, the gate and up halves meeting in LDS),
    tiles of 128 rows with a ring of three or two, or slabs through registers, by how many tiles there are; sizes
    that end inside a tile of rows and of columns."""
    rng = np.random.default_rng(47)
    a = bf(rng.standard_normal((M, K)).astype(np.float32))
    g, u = bf(rng.standard_normal((N, K)).astype(np.float32) * 0.1), bf(rng.standard_normal((N, K)).astype(np.float32) * 0.1)
    out = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    ops().gemm_swiglu(out, t(a, torch.bfloat16), t(g, torch.bfloat16), t(u, torch.bfloat16), kernel="tiled")
    close(out, pm.swiglu(pm.linear(a, g), pm.linear(a, u)), BF16, "gate/up")
    one = torch.empty(1, N, device=DEV, dtype=torch.bfloat16)
    ops().gemm_swiglu(one, t(a[M - 1:], torch.bfloat16), t(g, torch.bfloat16), t(u, torch.bfloat16), kernel="tiled")
    assert (one[0].float() - out[M - 1].float()).abs().max().item() <= 2e-2 * max(1.0, out[M - 1].float().abs().max().item())


def test_gate_up_of_few_rows_against_a_long_and_wide_pair_of_matrices():
    """The tiled gate/up form with 128 + 128 columns per block (192 such tiles or more, K from 2,048): sizes that end
    inside a tile, against a float32 product of the same operands."""
    o = ops()
    M, N, K = 37, 24700, 2112
    g = torch.Generator(device="cpu").manual_seed(3)
    a = torch.randn(M, K, generator=g).to(DEV, torch.bfloat16)
    wg, wu = (torch.randn(N, K, generator=g).mul_(0.05).to(DEV, torch.bfloat16) for _ in range(2))
    out = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
    o.gemm_swiglu(out, a, wg, wu, kernel="tiled")
    ref = torch.nn.functional.silu(a.float() @ wg.float().T) * (a.float() @ wu.float().T)
    err = ((out.float() - ref).abs().max() / ref.abs().max()).item()
    assert err < 1e-2, err


def test_few_rows_against_a_big_matrix_with_k_shared_out():
    """The tiled kernel with K shared out among blocks and the slabs straight into LDS: with few column tiles the
    shares are added by a second launch, with many (and weights of 32 MB or more) by the block of a tile that
    arrives last; a width that is no multiple of four takes neither. Sizes that end inside a tile and a share,
    residual and store epilogues, against a float32 product."""
    o = ops()
    g = torch.Generator(device="cpu").manual_seed(4)
    for M, N, K in ((40, 3600, 18944 + 64), (17, 1000, 2112), (64, 4608, 3584), (40, 5000, 3392), (33, 1001, 4160),
                    (1100, 896, 4864), (2000, 1000, 4160),       # many rows against a narrow matrix: tiles of 128 x 128, four and two shares
                    (100, 896, 4864), (250, 1000, 3136)):        # up to 256 rows: tiles of 64 x 128
        a = torch.randn(M, K, generator=g).to(DEV, torch.bfloat16)
        w = torch.randn(N, K, generator=g).mul_(0.05).to(DEV, torch.bfloat16)
        base = torch.randn(M, N, generator=g).to(DEV)
        acc = base.clone()
        o.gemm(acc, a, w, add_to_out=True, kernel="tiled")
        ref = a.float() @ w.float().T
        assert ((acc - base - ref).abs().max() / ref.abs().max()).item() < 1e-4, (M, N, K)
        bias = torch.randn(N, generator=g).to(DEV)
        out = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
        o.gemm(out, a, w, bias, kernel="tiled")
        assert ((out.float() - ref - bias).abs().max() / ref.abs().max()).item() < 1e-2, (M, N, K)
        out32 = torch.full((M, N), float("nan"), device=DEV)
        o.gemm(out32, a, w, kernel="tiled")
        assert ((out32 - ref).abs().max() / ref.abs().max()).item() < 1e-4, (M, N, K)
        again = base.clone()
        o.gemm(again, a, w, add_to_out=True, kernel="tiled")
        assert torch.equal(again, acc), (M, N, K)            # the shares are added in a fixed order


def test_many_rows_in_tiles_of_128_x_256():
    """The tiled kernel's widest tiles (128 x 256 and 128 x 192 for store and residual, 128 x (128 + 128) for gate/up;
    K from 2,048 and tile counts that fill rounds of the chip): sizes that end inside a tile, against a float32
    product."""
    o = ops()
    g = torch.Generator(device="cpu").manual_seed(6)
    M, N, K = 1990, 3600, 2112                 # 15 x 16 tiles of 128 x 256: 240 of 256
    a = torch.randn(M, K, generator=g).to(DEV, torch.bfloat16)
    w = torch.randn(N, K, generator=g).mul_(0.05).to(DEV, torch.bfloat16)
    ref = a.float() @ w.float().T
    out = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
    bias = torch.randn(N, generator=g).to(DEV)
    o.gemm(out, a, w, bias, kernel="tiled")
    assert ((out.float() - ref - bias).abs().max() / ref.abs().max()).item() < 1e-2
    base = torch.randn(M, N, generator=g).to(DEV)
    acc = base.clone()
    o.gemm(acc, a, w, add_to_out=True, kernel="tiled")
    assert ((acc - base - ref).abs().max() / ref.abs().max()).item() < 1e-4
    for M, N in ((1000, 3700), (1990, 5100)):  # tiles of 128 x 192: 8 x 20 in one round; 16 x 27 = 432 of 512
        a = torch.randn(M, K, generator=g).to(DEV, torch.bfloat16)
        w = torch.randn(N, K, generator=g).mul_(0.05).to(DEV, torch.bfloat16)
        ref = a.float() @ w.float().T
        out = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
        bias = torch.randn(N, generator=g).to(DEV)
        o.gemm(out, a, w, bias, kernel="tiled")
        assert ((out.float() - ref - bias).abs().max() / ref.abs().max()).item() < 1e-2
        base = torch.randn(M, N, generator=g).to(DEV)
        acc = base.clone()
        o.gemm(acc, a, w, add_to_out=True, kernel="tiled")
        assert ((acc - base - ref).abs().max() / ref.abs().max()).item() < 1e-4
    M, N = 1990, 3800                          # gate/up: 16 x 30 tiles of 128 x (128 + 128): 480 of 512
    a = torch.randn(M, K, generator=g).to(DEV, torch.bfloat16)
    wg, wu = (torch.randn(N, K, generator=g).mul_(0.05).to(DEV, torch.bfloat16) for _ in range(2))
    act = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
    o.gemm_swiglu(act, a, wg, wu, kernel="tiled")
    ref = torch.nn.functional.silu(a.float() @ wg.float().T) * (a.float() @ wu.float().T)
    assert ((act.float() - ref).abs().max() / ref.abs().max()).item() < 1e-2


def test_products_at_random_sizes():
    """Every form of the bfloat16 product (store with bias, float32 store, residual, gate/up, and the norm on the
    way in) through every kernel that takes the sizes (vector-unit, matrix-core for few rows, tiled, and the one
    the rule picks), at sizes drawn at random around the kernels' boundaries, against a float32 product of the
    same operands."""
    import random
    o = ops()
    rnd = random.Random(11)
    ran = {}
    for _ in range(150):
        M = rnd.choice([1, 2, 3, 5, 8, 9, 16, 17, 33, 64, 65, 130, 257, 520])
        N = rnd.choice([8, 35, 97, 200, 896, 1152, 2049])
        K = 8 * rnd.choice([1, 5, 16, 33, 64, 112, 193, 608, 770])
        kind = rnd.choice(["store", "float32 store", "residual", "gate/up", "norm + store", "norm + gate/up"])
        x = torch.randn(M, K, device=DEV)
        a = x.to(torch.bfloat16)
        w, w2 = (torch.randn(N, K, device=DEV).mul_(0.1).to(torch.bfloat16) for _ in range(2))
        bias, nw = torch.randn(N, device=DEV), torch.rand(K, device=DEV) + 0.5
        normed = (x * nw).to(torch.bfloat16).float() * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-5)
        for kernel in ("rows", "stream", "tiled", None):
            if kind.startswith("norm") and kernel == "tiled":
                continue
            try:
                if kind == "store":
                    out = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
                    o.gemm(out, a, w, bias, kernel=kernel)
                    ref = a.float() @ w.float().T + bias
                elif kind == "float32 store":
                    out = torch.full((M, N), float("nan"), device=DEV)
                    o.gemm(out, a, w, kernel=kernel)
                    ref = a.float() @ w.float().T
                elif kind == "residual":
                    base = torch.randn(M, N, device=DEV)
                    out = base.clone()
                    o.gemm(out, a, w, add_to_out=True, kernel=kernel)
                    ref = base + a.float() @ w.float().T
                elif kind == "gate/up":
                    out = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
                    o.gemm_swiglu(out, a, w, w2, kernel=kernel)
                    ref = torch.nn.functional.silu(a.float() @ w.float().T) * (a.float() @ w2.float().T)
                elif kind == "norm + store":
                    out = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
                    o.gemm(out, x, w, bias, kernel=kernel, norm=(nw, 1e-5))
                    ref = normed @ w.float().T + bias
                else:
                    out = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
                    o.gemm_swiglu(out, x, w, w2, kernel=kernel, norm=(nw, 1e-5))
                    ref = torch.nn.functional.silu(normed @ w.float().T) * (normed @ w2.float().T)
            except AlofaError:
                continue              # a kernel that does not take these sizes says so
            err = ((out.float() - ref).abs().max() / ref.abs().max().clamp_min(1e-6)).item()
            assert err < (1e-2 if out.dtype is torch.bfloat16 else 1e-4), f"{kind} through {kernel}: M={M} N={N} K={K} relative error {err}"
            ran[(kind, kernel)] = ran.get((kind, kernel), 0) + 1
    assert all(ran.get((kind, kernel), 0) > 0 for kind in ("store", "residual", "gate/up") for kernel in ("rows", "stream", "tiled", None)), ran


def test_gemm_with_operands_beyond_the_l2():
    """Operands of more than 32 MB make the tiled kernel deal its tiles out die by die (another
    numbering of the blocks): every tile must still be computed exactly once, with K shared out
    among blocks and with the SwiGLU epilogue too."""
    rng = np.random.default_rng(41)
    for M, N, K in [(130, 9000, 2048), (40, 1100, 16384)]:
        a, w = bf(rng.standard_normal((M, K)).astype(np.float32)), bf(rng.standard_normal((N, K)).astype(np.float32) * 0.05)
        res = rng.standard_normal((M, N)).astype(np.float32)
        acc = t(res)
        ops().gemm(acc, t(a, torch.bfloat16), t(w, torch.bfloat16), add_to_out=True, kernel="tiled")
        close(acc, pm.add(res, pm.linear(a, w)), 1e-4, f"residual {M}x{N}x{K}")
    M, N, K = 70, 4200, 2048
    a = bf(rng.standard_normal((M, K)).astype(np.float32))
    g, u = bf(rng.standard_normal((N, K)).astype(np.float32) * 0.03), bf(rng.standard_normal((N, K)).astype(np.float32) * 0.03)
    out = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    ops().gemm_swiglu(out, t(a, torch.bfloat16), t(g, torch.bfloat16), t(u, torch.bfloat16), kernel="tiled")
    close(out, pm.swiglu(pm.linear(a, g), pm.linear(a, u)), BF16, "swiglu")
