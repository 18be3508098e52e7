"""Each HIP kernel alone against a plain float32/float64 torch expression of the same op, at sizes
other than the engine's test models: widths and vocabularies that are no power of two, head sizes
in steps of 16, odd head counts and groups, rows that do not fill a tile."""

from __future__ import annotations

import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F32, BF16 = torch.float32, torch.bfloat16


@pytest.fixture(scope="module")
def ops():
    from miniserve_amd.kernels import ops as o

    o.library()
    return o


def rand(shape, dtype=F32, seed=0, scale=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * scale).to(dtype).to(DEV)


def close(got, want, rel, what=""):
    got, want = got.double().cpu(), want.double().cpu()
    scale = float(want.abs().max()) or 1.0
    err = float((got - want).abs().max())
    assert err <= rel * scale, f"{what}: max |diff| {err:.3e} > {rel * scale:.3e}"


# ------------------------------------------------------------------------------------------ elementwise


@pytest.mark.parametrize("table_dtype", [F32, BF16])
def test_embed(ops, table_dtype):
    table = rand((379, 96), table_dtype, 1)
    ids = torch.tensor([0, 378, 5, 5, 17], dtype=torch.int32, device=DEV)
    out = ops.embed(ids, table)
    assert out.dtype == F32
    assert torch.equal(out, table[ids.long()].float())


@pytest.mark.parametrize("width", [96, 1000, 5120])
@pytest.mark.parametrize("w_dtype,out_dtype", [(F32, F32), (BF16, BF16), (F32, BF16), (BF16, F32)])
def test_rmsnorm(ops, width, w_dtype, out_dtype):
    x = rand((7, width), F32, 2, 3.0)
    w = rand((width,), w_dtype, 3)
    eps = 1e-5
    xd = x.double()
    want = xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + eps) * w.double()
    got = ops.rmsnorm(x, w, eps, out_dtype)
    close(got, want, 1e-6 if out_dtype == F32 else 5e-3, "rmsnorm")
    rows = torch.tensor([6, 0, 3], dtype=torch.int32, device=DEV)
    got = ops.rmsnorm(x, w, eps, out_dtype, rows)
    close(got, want[rows.long()], 1e-6 if out_dtype == F32 else 5e-3, "rmsnorm rows")


@pytest.mark.parametrize("width,splits", [(96, 3), (1000, 11), (1024, 8), (5120, 16), (4098, 2)])
@pytest.mark.parametrize("out_dtype", [F32, BF16])
def test_rmsnorm_adds_partial_sums(ops, width, splits, out_dtype):
    """Every shape of the norm kernels (vector and scalar, one or several groups per thread, a number
    of splits that is no multiple of the load batch) adds the partial sums in full, with and without a
    row list."""
    m, eps = 5, 1e-6
    x = rand((m, width), F32, 60, 2.0)
    parts = rand((splits, m, width), F32, 61)
    w = rand((width,), BF16, 62) + 1
    full = x.double() + parts.double().sum(0)
    want = full / torch.sqrt((full * full).mean(-1, keepdim=True) + eps) * w.double()
    tol = 1e-5 if out_dtype == F32 else 5e-3
    x1 = x.clone()
    close(ops.rmsnorm(x1, w, eps, out_dtype, add=ops.SplitSum(parts)), want, tol, "all rows")
    close(x1, full, 1e-6, "stream brought up to date")
    x2 = x.clone()
    rows = torch.tensor([4, 1, 1], dtype=torch.int32, device=DEV)
    close(ops.rmsnorm(x2, w, eps, out_dtype, rows, add=ops.SplitSum(parts)), want[rows.long()], tol, "row list")
    assert torch.equal(x2, x)


def test_rmsnorm_eps_enters(ops):
    x = rand((2, 64), F32, 4, 1e-3)
    w = torch.ones(64, device=DEV)
    a, b = ops.rmsnorm(x, w, 1e-6, F32), ops.rmsnorm(x, w, 1e-5, F32)
    assert (a - b).abs().max() > 1e-2  # at this scale eps is of the size of mean(x^2)


def activation(name, g):
    """The gate's activation in float64, from its definition: silu(x) = x sigmoid(x); gelu_tanh is the
    tanh approximation of x Phi(x), x / 2 (1 + tanh(sqrt(2 / pi) (x + 0.044715 x^3)))."""
    if name == "silu":
        return g / (1 + torch.exp(-g))
    assert name == "gelu_tanh"
    return 0.5 * g * (1 + torch.tanh(math.sqrt(2 / math.pi) * (g + 0.044715 * g**3)))


def test_the_two_activations_are_not_each_other():
    g = torch.linspace(-6, 6, 49, dtype=torch.float64)
    phi = 0.5 * (1 + torch.erf(g / math.sqrt(2)))
    assert float((activation("gelu_tanh", g) - g * phi).abs().max()) < 5e-4  # the approximation of x Phi(x)
    assert float((activation("silu", g) - g * torch.sigmoid(g)).abs().max()) < 1e-15
    assert float((activation("silu", g) - activation("gelu_tanh", g)).abs().max()) > 0.1


@pytest.mark.parametrize("act", ["silu", "gelu_tanh"])
@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("inter", [224, 100, 3072])  # a multiple of 8 moves vectors, others single elements
def test_act_mul(ops, dtype, inter, act):
    gu = rand((5, 2 * inter), dtype, 5, 2.0)
    g, u = gu[:, :inter].double(), gu[:, inter:].double()
    want = activation(act, g) * u
    close(ops.act_mul(gu, act), want, 1e-6 if dtype == F32 else 5e-3, "act_mul")
    z = torch.zeros((1, 8), dtype=dtype, device=DEV)
    assert float(ops.act_mul(z, act).abs().max()) == 0.0
    if inter % 16 == 0:  # the same values with gates and ups in alternating runs of 16
        mixed = torch.stack((gu[:, :inter].reshape(5, inter // 16, 16), gu[:, inter:].reshape(5, inter // 16, 16)), dim=2)
        close(ops.act_mul(mixed.reshape(5, 2 * inter).contiguous(), act, block=16), want, 1e-6 if dtype == F32 else 5e-3, "runs of 16")
        parts = torch.stack([mixed.reshape(5, 2 * inter).float() * f for f in (0.5, 0.25, 0.25)])
        close(ops.act_mul(ops.SplitSum(parts), act, out_dtype=dtype, block=16), want, 1e-6 if dtype == F32 else 5e-3, "partial sums")
    with pytest.raises(NotImplementedError, match="gelu_tanh"):  # the message names what there is
        ops.act_mul(gu, "relu")


# (rows, width of x, outputs): up to 64 rows run one fused kernel whose waves split K and meet in LDS
# (K up to 2048 for up to 16 rows, up to 1024 for 17 to 64); many rows the tile kernels with the
# activation in their epilogue; more K at few rows, few tiles, a K that is no multiple of 64, or float32
# run the product and the activation as two kernels. All must agree.
GATED = [(3000, 128, 4096), (1, 1024, 3072), (8, 1024, 3072), (16, 512, 64), (5, 2048, 160), (13, 4096, 48), (40, 1024, 3072), (64, 256, 64),
         (17, 1024, 3072), (32, 768, 160), (33, 512, 48), (64, 1024, 3072), (50, 2048, 64),
         (200, 1024, 3072), (2048, 1024, 3072), (1000, 1024, 3072), (300, 192, 8192), (130, 96, 224), (9, 100, 48), (3000, 64, 4096),
         (2048, 512, 12288), (4090, 512, 4080)]
# The tile the activation's epilogue runs in, for the rows that are here for one (None: not asserted).
GATED_TILES = {(3000, 128, 4096): (128, 128), (200, 1024, 3072): (64, 64), (2048, 1024, 3072): (256, 256), (1000, 1024, 3072): (128, 192),
               (300, 192, 8192): (128, 64), (3000, 64, 4096): (128, 64),
               (2048, 512, 12288): (256, 256), (4090, 512, 4080): (256, 256)}  # the last: ragged in both directions


@pytest.mark.parametrize("act", ["silu", "gelu_tanh"])
@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("m,k,inter", GATED)
def test_gated_linear(ops, dtype, m, k, inter, act):
    x = rand((m, k), dtype, 70)
    gate, up = rand((inter, k), dtype, 71, 0.05), rand((inter, k), dtype, 72, 0.05)
    g, u = x.double() @ gate.double().T, x.double() @ up.double().T
    want = activation(act, g) * u
    w = ops.interleave_gate_up(gate, up)
    assert w.shape == (2 * inter, k) and torch.equal(w[:16], gate[:16]) and torch.equal(w[16:32], up[:16])
    if (m, k, inter) in GATED_TILES:
        assert ops.tile_shape(m, 2 * inter, k, gated=True) == GATED_TILES[(m, k, inter)], "pick other sizes for this tile shape"
    got = ops.gated_linear(x, w, act, out_dtype=dtype, block=ops.GATE_BLOCK)
    assert got.shape == (m, inter) and got.dtype == dtype
    close(got, want, 1e-5 if dtype == F32 else 8e-3, f"gated {m}x{k}->{inter}")
    # and with the plain layout (gates, then ups) through the two-kernel path
    close(ops.gated_linear(x, torch.cat((gate, up)).contiguous(), act, out_dtype=dtype), want, 1e-5 if dtype == F32 else 8e-3, "halves")


# ------------------------------------------------------------------------------------------ matrix products


@pytest.mark.parametrize("m,n,k", [(1, 64, 64), (5, 379, 96), (130, 200, 224), (64, 70, 37), (3, 1024, 3072)])
def test_gemm_f32(ops, m, n, k):
    x, w = rand((m, k), F32, 6), rand((n, k), F32, 7)
    want = x.double() @ w.double().T
    close(ops.linear(x, w, out_dtype=F32), want, 2e-6, "gemm f32")
    acc = rand((m, n), F32, 8)
    before = acc.clone()
    ops.linear(x, w, accumulate_into=acc)
    close(acc, before.double() + want, 2e-6, "gemm f32 accumulate")
    close(ops.linear(x, w, out_dtype=BF16), want, 5e-3, "gemm f32 -> bf16")


def test_gemm_f32_rows_do_not_depend_on_batch(ops):
    x, w = rand((130, 224), F32, 9), rand((379, 224), F32, 10)
    whole = ops.linear(x, w, out_dtype=F32)
    for lo, hi in ((0, 1), (63, 66), (100, 130)):
        assert torch.equal(ops.linear(x[lo:hi].contiguous(), w, out_dtype=F32), whole[lo:hi])


@pytest.mark.parametrize("m", [1, 7, 16, 17, 33, 64, 65, 200, 1000])
@pytest.mark.parametrize("n,k", [(379, 96), (192, 224), (1024, 1024), (100, 100), (4096, 128)])
def test_gemm_bf16(ops, m, n, k):
    x, w = rand((m, k), BF16, 11), rand((n, k), BF16, 12)
    want = x.double() @ w.double().T
    close(ops.linear(x, w, out_dtype=F32), want, 1e-5, f"gemm bf16 {m}x{n}x{k} -> f32")
    close(ops.linear(x, w, out_dtype=BF16), want, 5e-3, "gemm bf16 -> bf16")
    acc = rand((m, n), F32, 13)
    before = acc.clone()
    ops.linear(x, w, accumulate_into=acc)
    close(acc, before.double() + want, 1e-5, "gemm bf16 accumulate")


@pytest.mark.parametrize("m,n,k,tile", [
    # a short K: the fixed part of the time decides, 128 x 64 tiles; edge tiles in both directions, one slab, an odd number of slabs
    (2000, 2100, 192, (128, 64)), (4100, 1000, 64, (128, 64)), (300, 14000, 320, (128, 64)), (4000, 1500, 192, (128, 64)),
    (2048, 6100, 128, (128, 64)), (5000, 5000, 128, (128, 64)), (4096, 4096, 64, (128, 64)),
    (2048, 4096, 1024, (128, 128)), (600, 33000, 192, (128, 128)),
    # fewer than 256 tiles of 128 x 128: 64 x 64 tiles of the same kernel
    (1990, 1000, 128, (64, 64)), (2048, 1000, 256, (64, 64)),
    # 128 x 160 (32 columns of tiles, the last one cut off, exactly 512 tiles; and 33 rows of 7 tiles)
    (1990, 5100, 512, (128, 160)), (4100, 1000, 512, (128, 160)),
    # 128 x 192 (many rows, and few rows of a wide matrix)
    (4000, 4200, 1024, (128, 192)), (600, 33000, 512, (128, 192)),
    # 256 x 256 tiles of four waves, one block per CU taking tiles in turn (exactly 256 with both edges ragged, and 240 tiles)
    (4090, 4090, 1024, (256, 256)), (3000, 5000, 1024, (256, 256)),
    # the same with the fewest slabs its loop takes (two), with three, and two rounds of tiles with five slabs
    (4000, 4088, 128, (256, 256)), (2048, 8192, 192, (256, 256)), (4096, 8192, 320, (256, 256)),
])
def test_gemm_bf16_large_tiles(ops, m, n, k, tile):
    """Every tile shape of the kernel whose slabs go straight into LDS (K a multiple of 64). Which shape a
    product takes follows a fitted time model; the library says which it picks, and a row whose sizes no
    longer reach the shape it is here for fails instead of testing another shape twice. Rows past the end
    are read from the last valid row and never stored."""
    assert ops.tile_shape(m, n, k) == tile, "this row no longer reaches the tile shape it was chosen for: pick other sizes"
    x, w = rand((m, k), BF16, 14), rand((n, k), BF16, 15)
    want = x.double() @ w.double().T
    close(ops.linear(x, w, out_dtype=F32), want, 1e-5, f"gemm bf16 {m}x{n}x{k} -> f32")
    close(ops.linear(x, w, out_dtype=BF16), want, 5e-3, "gemm bf16 -> bf16")
    acc = rand((m, n), F32, 16)
    before = acc.clone()
    ops.linear(x, w, accumulate_into=acc)
    close(acc, before.double() + want, 1e-5, "gemm bf16 accumulate")


def _wide_tile_draws(seed):
    """Sizes drawn at random (a fixed seed): rows and columns with ragged edges, K from two slabs on, plain and gated."""
    import random
    rng = random.Random(seed)
    while True:
        m = rng.choice([rng.randint(257, 5000), rng.choice([512, 1024, 2048, 4096])])
        n = rng.choice([rng.randint(32, 800) * 8, rng.choice([4096, 5120, 6144])])
        k = rng.choice([128, 192, 256, 320, 1024, 2048, 4160]) if rng.random() < 0.7 else rng.randint(2, 60) * 64
        gated = rng.random() < 0.3
        yield m, (n // 32 * 32 if gated else n), k, gated


@pytest.mark.parametrize("seed", [0, 1])
def test_wide_tile_at_random_sizes(ops, seed):
    """The four-wave 256 x 256 tile, whose loop is written in assembly, at sizes nobody chose: every output
    form (bfloat16, float32, added into a float32 matrix, partial sums of a split K, gated with both
    activations) against float64, and twice for equal bits (a tile taken by another block, in another turn,
    must give the same)."""
    lib = ops.library()
    done = 0
    for tries, (m, n, k, gated) in enumerate(_wide_tile_draws(seed)):
        if done == 8 or tries == 4000:
            break
        if m * n > 24e6 or (m + n) * k > 60e6:
            continue
        splits = 1 if gated else lib.ms_gemm_bf16_tile_splits(m, n, k)
        if ops.tile_shape(m, n, k, splits, gated) != (256, 256):
            continue
        done += 1
        what = f"{m}x{n}x{k} splits {splits} gated {gated}"
        x, w = rand((m, k), BF16, 300 + done), rand((n, k), BF16, 400 + done, 0.05)
        want = x.double() @ w.double().T
        if gated:
            pairs = want.view(m, n // 32, 2, 16)
            g, u = pairs[:, :, 0].reshape(m, n // 2), pairs[:, :, 1].reshape(m, n // 2)
            for act in ("silu", "gelu_tanh"):
                a = ops.gated_linear(x, w, act, out_dtype=BF16, block=ops.GATE_BLOCK)
                close(a, activation(act, g) * u, 8e-3, f"{what} {act}")
                assert torch.equal(a, ops.gated_linear(x, w, act, out_dtype=BF16, block=ops.GATE_BLOCK)), what
            continue
        a = ops.linear(x, w, out_dtype=BF16)
        close(a, want, 5e-3, f"{what} -> bf16")
        assert torch.equal(a, ops.linear(x, w, out_dtype=BF16)), what
        close(ops.linear(x, w, out_dtype=F32), want, 1e-5, f"{what} -> f32")
        acc = rand((m, n), F32, 500 + done)
        before = acc.clone()
        pend = ops.linear(x, w, accumulate_into=acc, defer=True)
        if pend is not None:
            assert pend.splits == splits, what
            ops.add_pending(acc, pend)
        close(acc.double() - before.double(), want, 1e-5, f"{what} accumulate")
    assert done == 8, "the draw no longer reaches the 256 x 256 tile often enough: widen it"


@pytest.mark.parametrize("m", [1, 8, 16, 40, 64])
def test_pending_sums_feed_their_consumers(ops, m):
    """The small-M product may leave partial sums for the next kernel to add: every consumer of such
    a sum gives what it gives on the finished matrix."""
    k, n = 1024, 1024
    x, w = rand((m, k), BF16, 50), rand((n, k), BF16, 51, 0.05)
    want = x.double() @ w.double().T
    s = ops.linear(x, w, out_dtype=BF16, defer=True)
    assert isinstance(s, ops.SplitSum) and s.splits > 1 and s.shape == (m, n)
    close(s.parts.sum(0), want, 1e-5, "partial sums")
    # the number of splits depends on the matrix and on the class of the row count (up to 4, 5 to 16, more), not on the rows themselves
    other = x[:1] if m <= 4 else (torch.cat([x, x])[:5] if m <= 16 else torch.cat([x, x])[:17])
    assert ops.linear(other.contiguous(), w, out_dtype=BF16, defer=True).splits == s.splits
    # residual stream: norm with the pending sum added first, rows or all
    resid = rand((m, n), F32, 52)
    nw = rand((n,), BF16, 53) + 1
    full = resid.double() + want
    normed = full / torch.sqrt((full * full).mean(-1, keepdim=True) + 1e-6) * nw.double()
    r1 = resid.clone()
    pend = ops.linear(x, w, accumulate_into=r1, defer=True)
    assert isinstance(pend, ops.SplitSum) and torch.equal(r1, resid)  # nothing was added yet
    close(ops.rmsnorm(r1, nw, 1e-6, BF16, add=pend), normed, 5e-3, "norm with pending sum")
    close(r1, full, 1e-5, "residual brought up to date")
    r2 = resid.clone()
    rows = torch.tensor([m - 1, 0, 0], dtype=torch.int32, device=DEV)  # a row may be asked for twice
    close(ops.rmsnorm(r2, nw, 1e-6, F32, rows, add=pend), normed[rows.long()], 1e-5, "norm of rows with pending sum")
    assert torch.equal(r2, resid)  # with a row list the stream itself is left alone
    r3 = resid.clone()
    ops.add_pending(r3, pend)
    close(r3, full, 1e-5, "add_pending")
    # gated activation
    gu = ops.linear(x, w, out_dtype=BF16, defer=True)
    g, u = want[:, : n // 2], want[:, n // 2 :]
    close(ops.act_mul(gu, out_dtype=BF16), activation("silu", g) * u, 6e-3, "act_mul of partial sums")
    # without defer the same call returns the finished matrix / adds it
    close(ops.linear(x, w, out_dtype=F32), want, 1e-5, "finished matrix")
    r4 = resid.clone()
    assert ops.linear(x, w, accumulate_into=r4) is None
    close(r4, full, 1e-5, "accumulate")


@pytest.mark.parametrize("n,k", [(4112, 4096), (33000, 520), (4111, 4096)])
def test_small_product_with_shared_rows_on_large_matrices(ops, n, k):
    """Above 16 M weights and from 4 rows on, the product for up to 16 rows stages its rows in LDS for
    four waves (N no multiple of 64: the last block has waves without weight rows; K = 520: a slab that
    is cut off; N = 4111: rows of partial sums that are not 16-byte aligned). Both forms add the same products in the same order: a row gives the same bits alone."""
    x, w = rand((16, k), BF16, 70), rand((n, k), BF16, 71, 0.05)
    want = x.double() @ w.double().T
    rows = {}
    for m in (1, 3, 4, 9, 16):
        s = ops.linear(x[:m].contiguous(), w, out_dtype=BF16, defer=True)
        assert isinstance(s, ops.SplitSum)
        rows[m] = s.parts.clone()
        close(rows[m].sum(0), want[:m], 1e-5, f"{m} rows of {n}x{k}")
    for m in (3, 4, 9, 16):
        assert torch.equal(rows[m][:, :1], rows[1])
    assert torch.equal(rows[16][:, :9], rows[9])


@pytest.mark.parametrize("m,n,k,cols", [(40, 32776, 4096, 128), (17, 24680, 5440, 128), (64, 51200, 4096, 256), (33, 40968, 5120, 256)])
def test_products_of_17_to_64_rows_take_wider_tiles_on_large_matrices(ops, m, n, k, cols):
    """From 224 MB of weights on the tiles of a 17- to 64-row product are 128 columns wide, from 400 MB on
    256 (the library says which): other instances of the tile kernel than the 64 x 64 one that smaller
    matrices take. N no multiple of the tile's width, an odd number of slabs, K split or not."""
    lib = ops.library()
    assert lib.ms_gemm_bf16_small_tile_cols(n, k) == cols, "pick other sizes for this tile width"
    x, w = rand((m, k), BF16, 80), rand((n, k), BF16, 81, 0.05)
    want = x.double() @ w.double().T
    s = ops.linear(x, w, out_dtype=BF16, defer=True)
    assert isinstance(s, ops.SplitSum) and s.splits == lib.ms_gemm_bf16_small_splits(m, n, k)
    close(s.parts.sum(0), want, 1e-5, f"partial sums of {m}x{n}x{k}")
    close(ops.linear(x, w, out_dtype=BF16), want, 5e-3, "finished matrix")
    one = ops.linear(x[:1].contiguous(), w, out_dtype=F32)
    close(one, want[:1], 1e-5, "one row of the same matrix (the small-M kernel)")


@pytest.mark.parametrize("m,n,k,splits", [(200, 1024, 2048, 8), (2048, 1024, 3072, 2), (300, 1000, 1100, 6), (2048, 4096, 1024, 1),
                                          (96, 6144, 4096, 8), (384, 4096, 4096, 4), (130, 1024, 1088, 6),
                                          (1024, 4096, 12288, 4), (768, 5120, 8192, 4), (2048, 4096, 8384, 2), (4000, 2048, 8256, 2),
                                          (500, 5120, 25600, 6)])
def test_tile_product_splits_k_when_tiles_are_few(ops, m, n, k, splits):
    """The last four have 256 and more tiles of 128 x 128 already: above 512 rows the splits follow the
    predicted time (a long K in parts makes 256 x 256 tiles enough to give every CU one), not the tile
    count alone. The very last two have a last split that is one slab shorter than the others, with an
    odd and an even number of slabs; the last one is a large matrix at under 512 rows, which takes many
    short splits for the same reason."""
    x, w = rand((m, k), BF16, 60), rand((n, k), BF16, 61, 0.05)
    want = x.double() @ w.double().T
    resid = rand((m, n), F32, 62)
    r = resid.clone()
    pend = ops.linear(x, w, accumulate_into=r, defer=True)
    if splits == 1:
        assert pend is None
    else:
        assert isinstance(pend, ops.SplitSum) and pend.splits == splits and torch.equal(r, resid)
        ops.add_pending(r, pend)
    close(r, resid.double() + want, 1e-5, "tile product with split K")


def test_linear_with_float32_weights_in_bfloat16_mode(ops):
    x, w = rand((9, 96), BF16, 14), rand((50, 96), F32, 15)
    close(ops.linear(x, w, out_dtype=BF16), x.double() @ w.double().T, 5e-3, "f32 weights, bf16 activations")


# ------------------------------------------------------------------------------------------ attention pieces


def plain_rope(x, pos, inv_freq, rot):
    """x [T, heads, D] float64; pairs (j, j + rot/2) of the first rot elements."""
    ang = pos.float()[:, None] * inv_freq[None, :]  # float32 as the engine forms it
    ang = ang.double()
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    half = rot // 2
    a, b = x[..., :half], x[..., half:rot]
    out = x.clone()
    out[..., :half] = a * cos - b * sin
    out[..., half:rot] = b * cos + a * sin
    return out


def test_rope_table(ops):
    pos = torch.tensor([0, 1, 2, 77, 4095, 40000], dtype=torch.int32, device=DEV)
    inv_freq = (1.0 / (1e6 ** (torch.arange(0, 48, 2).float() / 48))).to(DEV)
    table = ops.rope_table(pos, inv_freq)
    ang = (pos.float()[:, None] * inv_freq[None, :]).double()  # the angle itself is a float32 product
    assert table.shape == (6, 48) and table.dtype == F32
    close(table[:, :24], torch.cos(ang), 1e-6, "cosines")
    close(table[:, 24:], torch.sin(ang), 1e-6, "sines")
    assert torch.equal(table[0, :24], torch.ones(24, device=DEV)) and torch.equal(table[0, 24:], torch.zeros(24, device=DEV))


# (tokens, layout of the slots): few tokens run the kernel with a wave per head, many the tiled one,
# whose value store takes whole aligned runs of a page with one vector and everything else singly; above
# 256 tokens a block of the tiled kernel takes four heads of a kind.
QK_CASES = [(11, "scattered"), (150, "scattered"), (150, "runs"), (200, "shifted"), (300, "runs"), (333, "shifted")]


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("t,layout", QK_CASES)
@pytest.mark.parametrize("hq,hkv,d,rot,page", [(4, 2, 16, 16, 16), (6, 1, 32, 32, 16), (3, 3, 48, 24, 8), (5, 5, 256, 256, 4),
                                               (16, 8, 128, 128, 16), (3, 1, 64, 64, 16), (2, 2, 128, 0, 8), (4, 2, 64, 32, 16)])
def test_qk_norm_rope_store(ops, dtype, hq, hkv, d, rot, page, t, layout):
    pages, eps = (t + page - 1) // page + 9, 1e-5
    qkv = rand((t, (hq + 2 * hkv) * d), dtype, 16)
    qw, kw = rand((d,), dtype, 17) + 1, rand((d,), dtype, 18) + 1
    pos = torch.tensor(([0, 1, 2, 3, 40, 41, 700, 5, 6, 7, 4000] * 40)[:t], dtype=torch.int32, device=DEV)
    if layout == "scattered":
        perm = torch.randperm(pages * page, generator=torch.Generator().manual_seed(1))[:t]
    elif layout == "runs":  # consecutive slots from a page's start, as a prompt's portion has them
        perm = torch.arange(t) + 2 * page
    else:  # consecutive, but starting in the middle of a page and with a jump to another page
        second = (93 // page + 3) * page + 5
        perm = torch.cat([torch.arange(3, 3 + 90), torch.arange(second, second + t - 90)])
    slots = perm.to(torch.int32).to(DEV)
    inv_freq = (1.0 / (1e4 ** (torch.arange(0, rot, 2).float() / max(rot, 1)))).to(DEV)
    rope = ops.rope_table(pos, inv_freq) if rot else None
    kc = torch.full((pages, hkv, page, d), 7.0, dtype=dtype, device=DEV)
    vc = torch.full((pages, hkv, d, page), 7.0, dtype=dtype, device=DEV)  # values lie transposed within the page
    ref = qkv.double().view(t, hq + 2 * hkv, d)
    q, k, v = ref[:, :hq], ref[:, hq : hq + hkv], ref[:, hq + hkv :]

    def norm(x, w):
        return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w.double()

    qn = plain_rope(norm(q, qw), pos, inv_freq, rot) if rot else norm(q, qw)
    kn = plain_rope(norm(k, kw), pos, inv_freq, rot) if rot else norm(k, kw)
    work = qkv.clone()
    ops.qk_norm_rope_store(work, slots, qw, kw, eps, rope, kc, vc, hq, hkv, d)
    tol = 2e-6 if dtype == F32 else 5e-3
    close(work.view(t, hq + 2 * hkv, d)[:, :hq], qn, tol, "q")
    sl = slots.long()
    got_k = kc.permute(0, 2, 1, 3).reshape(pages * page, hkv, d)
    got_v = vc.permute(0, 3, 1, 2).reshape(pages * page, hkv, d)
    close(got_k[sl], kn, tol, "k in cache")
    assert torch.equal(got_v[sl].double(), v), "v is stored as it is"
    untouched = torch.ones(pages * page, dtype=torch.bool)
    untouched[sl.cpu()] = False
    assert float((got_k[untouched.to(DEV)] - 7).abs().max()) == 0 and float((got_v[untouched.to(DEV)] - 7).abs().max()) == 0
    # position 0 is the identity of the rotation
    close(work.view(t, hq + 2 * hkv, d)[0, :hq], norm(q, qw)[0], tol, "position 0")
    # the same from partial sums of qkv: queries come back in a tensor of their own
    parts = torch.stack([qkv.float() * 0.25, qkv.float() * 0.5, qkv.float() * 0.25])
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    q2 = ops.qk_norm_rope_store(ops.SplitSum(parts), slots, qw, kw, eps, rope, kc2, vc2, hq, hkv, d, out_dtype=dtype)
    assert q2.shape == (t, hq * d)
    close(q2.view(t, hq, d), qn, tol, "q from partial sums")
    close(kc2.permute(0, 2, 1, 3).reshape(pages * page, hkv, d)[sl], kn, tol, "k from partial sums")


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("hq,hkv,d,rot", [(4, 2, 16, 16), (3, 1, 64, 64), (16, 8, 128, 128), (5, 5, 48, 20), (2, 1, 256, 64)])
def test_qk_norm_rope_store_turns_adjacent_elements(ops, dtype, hq, hkv, d, rot):
    """The other pairing: elements (2j, 2j + 1) of a head are turned by angle j. Head sizes 64 and 128 take the
    wave-per-head kernel here too (the tiled one knows halves only); a pairing no kernel knows is refused."""
    t, page, eps = 70, 16, 1e-5
    pages = t // page + 3
    qkv = rand((t, (hq + 2 * hkv) * d), dtype, 26)
    qw, kw = rand((d,), dtype, 27) + 1, rand((d,), dtype, 28) + 1
    pos = torch.tensor(([0, 1, 2, 3, 40, 41, 700, 5, 6, 4000] * 7)[:t], dtype=torch.int32, device=DEV)
    slots = torch.randperm(pages * page, generator=torch.Generator().manual_seed(2))[:t].to(torch.int32).to(DEV)
    inv_freq = (1.0 / (1e4 ** (torch.arange(0, rot, 2).float() / rot))).to(DEV)
    rope = ops.rope_table(pos, inv_freq)
    kc, vc = torch.zeros((pages, hkv, page, d), dtype=dtype, device=DEV), torch.zeros((pages, hkv, d, page), dtype=dtype, device=DEV)
    ref = qkv.double().view(t, hq + 2 * hkv, d)

    def norm(x, w):
        return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w.double()

    def turn(x):
        ang = (pos.float()[:, None] * inv_freq[None, :]).double()
        cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        out = x.clone()
        a, b = x[..., 0:rot:2], x[..., 1:rot:2]
        out[..., 0:rot:2], out[..., 1:rot:2] = a * cos - b * sin, b * cos + a * sin
        return out

    work = qkv.clone()
    ops.qk_norm_rope_store(work, slots, qw, kw, eps, rope, kc, vc, hq, hkv, d, pairing="adjacent")
    tol = 2e-6 if dtype == F32 else 5e-3
    close(work.view(t, hq + 2 * hkv, d)[:, :hq], turn(norm(ref[:, :hq], qw)), tol, "q, adjacent pairs")
    got_k = kc.permute(0, 2, 1, 3).reshape(pages * page, hkv, d)
    close(got_k[slots.long()], turn(norm(ref[:, hq : hq + hkv], kw)), tol, "k in cache, adjacent pairs")
    if rot == d:  # and it is another rotation than that of the halves
        halves = qkv.clone()
        ops.qk_norm_rope_store(halves, slots, qw, kw, eps, rope, torch.zeros_like(kc), torch.zeros_like(vc), hq, hkv, d)
        assert float((halves.float() - work.float()).abs().max()) > 0.1
    with pytest.raises(NotImplementedError, match="pairing"):
        ops.qk_norm_rope_store(work, slots, qw, kw, eps, rope, kc, vc, hq, hkv, d, pairing="quarters")
    # the fused decode step takes halves only and says so
    batch = make_batch([1] * t, pos.tolist())
    parts = ops.SplitSum(torch.stack([qkv.float()]))
    if dtype == BF16 and d in (64, 128) and rot == d:
        assert ops.decode_attention_fusable(parts, batch, qw, kw, rope, kc, vc, hq, hkv, d)
        assert not ops.decode_attention_fusable(parts, batch, qw, kw, rope, kc, vc, hq, hkv, d, "adjacent")


class _Batch:
    def prefill_tiles(self, tile_tokens):
        from miniserve_amd.kernels.ops import build_prefill_tiles

        return build_prefill_tiles(self.row_lens, self.row_starts_host, tile_tokens, DEV)


def make_batch(lens_new, starts):
    batch = _Batch()
    batch.num_rows = len(lens_new)
    batch.token_row = torch.tensor([i for i, n in enumerate(lens_new) for _ in range(n)], dtype=torch.int32, device=DEV)
    batch.positions = torch.tensor([s + j for s, n in zip(starts, lens_new) for j in range(n)], dtype=torch.int32, device=DEV)
    batch.max_kv_len = max(s + n for s, n in zip(starts, lens_new))
    batch.row_lens, batch.row_starts_host = list(lens_new), list(starts)
    n_dec = sum(1 for n in lens_new if n == 1)
    batch.num_decode_tokens = n_dec
    batch.is_decode = n_dec == len(lens_new)
    batch.decode_tokens = batch.prefill_tokens = None
    if 0 < n_dec < len(lens_new):
        dec, pre, t = [], [], 0
        for n in lens_new:
            (dec if n == 1 else pre).extend(range(t, t + n))
            t += n
        batch.decode_tokens = torch.tensor(dec, dtype=torch.int32, device=DEV)
        batch.prefill_tokens = torch.tensor(pre, dtype=torch.int32, device=DEV)
    return batch


def attention_case(ops, dtype, hq, hkv, d, page, lens_new, starts, window, seed=0, boost=None):
    """Rows with ``starts[i]`` cached tokens and ``lens_new[i]`` new ones; scattered pages.
    ``boost = (row, position)``: the key there and the row's last query are scaled so that this
    one score stands out among all others (a far key that is skipped or misplaced then shows)."""
    g = torch.Generator().manual_seed(seed)
    b = len(lens_new)
    totals = [s + n for s, n in zip(starts, lens_new)]
    blocks = [-(-tt // page) for tt in totals]
    pages = sum(blocks) + 3
    order = torch.randperm(pages, generator=g).tolist()
    width = max(blocks)
    table = torch.full((b, width), -1, dtype=torch.int32)
    kc = rand((pages, hkv, page, d), dtype, seed + 1)
    vc = rand((pages, hkv, d, page), dtype, seed + 2)
    at = 0
    for i, nb in enumerate(blocks):
        table[i, :nb] = torch.tensor(order[at : at + nb], dtype=torch.int32)
        at += nb
    t = sum(lens_new)
    q = rand((t, (hq + 2 * hkv) * d), dtype, seed + 3)
    if boost is not None:
        row, where = boost
        last = sum(lens_new[: row + 1]) - 1
        key = kc[table[row, where // page], :, where % page]  # [hkv, d]
        qv = q[last].view(hq + 2 * hkv, d)
        for h in range(hq):
            qv[h] = (key[h // (hq // hkv)].float() * 3.0).to(dtype)
    batch = make_batch(lens_new, starts)
    scale = d**-0.5
    got = ops.paged_attention(q, kc, vc, table.to(DEV), batch, hq, hkv, d, scale, window)
    want = torch.empty((t, hq, d), dtype=torch.float64)
    qd = q.double().cpu().view(t, hq + 2 * hkv, d)[:, :hq]
    kcd, vcd = kc.double().cpu(), vc.double().cpu()
    tok = 0
    for i in range(b):
        keys = torch.stack([kcd[table[i, p // page], :, p % page] for p in range(totals[i])])  # [len, hkv, d]
        vals = torch.stack([vcd[table[i, p // page], :, :, p % page] for p in range(totals[i])])
        for j in range(lens_new[i]):
            p = starts[i] + j
            lo = max(0, p - window + 1) if window else 0
            for h in range(hq):
                kh = h // (hq // hkv)
                s = (keys[lo : p + 1, kh] @ qd[tok, h]) * scale
                w = torch.softmax(s, 0)
                if boost is not None and boost[0] == i and j == lens_new[i] - 1 and lo <= boost[1] <= p:
                    assert float(w[boost[1] - lo]) > 0.9, "the boosted key was meant to dominate"
                want[tok, h] = w @ vals[lo : p + 1, kh]
            tok += 1
    close(got.view(t, hq, d), want, 2e-6 if dtype == F32 else 8e-3, f"attention {hq}/{hkv}/{d} window {window}")


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize(
    "hq,hkv,d,page,lens_new,starts,window",
    [
        (4, 2, 16, 16, [5, 1, 40], [0, 17, 3], 0),
        (6, 1, 32, 16, [1, 1, 1, 1], [0, 15, 16, 130], 0),
        (3, 3, 48, 8, [70, 2], [0, 100], 24),
        (16, 8, 128, 16, [33, 1], [31, 200], 0),
        (5, 5, 256, 4, [3, 9], [64, 0], 7),
        (8, 2, 64, 16, [130], [0], 0),
    ],
)
def test_paged_attention(ops, dtype, hq, hkv, d, page, lens_new, starts, window):
    attention_case(ops, dtype, hq, hkv, d, page, lens_new, starts, window)


@pytest.mark.parametrize(
    "hq,hkv,d,lens_new,starts,window,boost",
    [
        (16, 8, 128, [1] * 7, [0, 15, 16, 31, 32, 1000, 4095], 0, None),   # page and chunk edges, many splits
        (16, 8, 128, [1, 1], [700, 3000], 0, (1, 37)),                     # a far key among thousands
        (16, 8, 128, [1, 1], [700, 3000], 0, (0, 699)),                    # the newest cached key
        (32, 8, 128, [1] * 3, [5, 260, 90], 0, (1, 255)),
        (64, 8, 128, [1] * 2, [513, 77], 0, None),
        (14, 2, 64, [1] * 5, [63, 64, 65, 2000, 1], 0, (3, 1024)),
        (6, 6, 64, [1] * 4, [300, 40, 41, 1200], 100, (0, 201)),           # the window's first key
        (16, 8, 128, [1] * 3, [500, 31, 2047], 33, (2, 2047 - 33 + 1)),
        (16, 8, 128, [1, 20, 1, 5, 1], [100, 0, 1999, 30, 0], 0, (2, 3)),  # decode rows beside portions
        (4, 2, 128, [1] * 64, list(range(0, 6400, 100)), 0, None),         # a full batch: one split
    ],
)
def test_decode_attention_bf16(ops, hq, hkv, d, lens_new, starts, window, boost):
    attention_case(ops, BF16, hq, hkv, d, 16, lens_new, starts, window, seed=30, boost=boost)


@pytest.mark.parametrize(
    "hq,hkv,d,lens_new,starts,window,boost",
    [
        (16, 8, 128, [200], [0], 0, (0, 5)),                          # a whole prompt, several tiles
        (16, 8, 128, [64, 65, 2], [0, 0, 0], 0, None),                # a full tile, one token more, the shortest portion
        (16, 8, 128, [70], [1000], 0, (0, 17)),                       # a portion deep into a sequence, a far key
        (16, 8, 128, [33, 1, 90, 1], [31, 200, 64, 0], 0, (2, 63)),   # portions beside decode rows
        (32, 8, 128, [50, 40], [10, 300], 0, (1, 299)),               # four heads per group: 32 tokens per tile
        (64, 8, 128, [40], [100], 0, (0, 3)),                         # eight heads per group
        (14, 2, 64, [100, 3], [0, 77], 0, (0, 50)),                   # seven heads per group: 18 tokens per tile, rows idle
        (6, 6, 64, [150], [20], 0, None),                             # one head per group: 128 tokens per tile
        (16, 8, 128, [150, 30], [0, 500], 40, (0, 149 - 39)),         # a window: its first key stands out
        (16, 8, 128, [130], [300], 200, (0, 230)),                    # a window wider than the tile
        (6, 6, 64, [300], [0], 17, None),                             # a window narrower than a key tile
        (16, 8, 128, [700], [0], 0, (0, 100)),                        # deep tiles' keys in parts: a key of an early part
        (16, 8, 128, [300, 1], [900, 50], 0, (0, 1199 - 70)),         # parts beside a decode row: a key of the last but one part
        (8, 2, 64, [500, 40], [0, 0], 0, (0, 3)),                     # head size 64, whole tiles beside tiles in parts
        (16, 8, 128, [64, 1], [6000, 9], 0, (0, 4000)),               # a short portion far into a sequence: parts by the host's own rule
    ],
)
@pytest.mark.parametrize("parts", ["host rule", "wherever possible"])
@pytest.mark.parametrize("tile_rows", [64, 128])
def test_prefill_attention_bf16(ops, monkeypatch, hq, hkv, d, lens_new, starts, window, boost, parts, tile_rows):
    """``parts``: the keys of deep tiles are handed out in parts where the host's estimate says it pays, or
    (second run) wherever a tile is deeper than the shortest part, so that small cases take that path too.
    ``tile_rows``: 64 query rows per block, as steps of this size run by themselves, or the 128-row blocks
    (two wave groups that share a key tile and own 64 query rows each) that long steps take, forced here
    by setting the number of blocks from which they run to zero."""
    if parts == "wherever possible":
        monkeypatch.setattr(ops, "PREFILL_PARTS_LAUNCH_US", -1e9)
    if tile_rows == 128:
        monkeypatch.setattr(ops, "PREFILL_BIG_BLOCKS", 0)
    seen = spy_prefill_rows(ops, monkeypatch)
    attention_case(ops, BF16, hq, hkv, d, 16, lens_new, starts, window, seed=40, boost=boost)
    assert seen == [tile_rows], seen


def spy_prefill_rows(ops, monkeypatch) -> list:
    """Records the query rows per block of every launch of the prefill attention."""
    lib, seen = ops.library(), []
    for name, at in (("ms_attention_prefill_bf16", 9), ("ms_attention_prefill_parts_bf16", 11)):
        real = getattr(lib, name)

        def wrapped(*args, _real=real, _at=at):
            seen.append(args[_at])
            return _real(*args)

        monkeypatch.setattr(lib, name, wrapped)
    return seen


@pytest.mark.parametrize(
    "hq,hkv,d,lens_new,starts,boost",
    [
        (64, 8, 128, [1300], [0], (0, 70)),            # a step long enough for 128-row blocks by its own size
        (16, 8, 128, [5200, 1], [40, 3000], (0, 11)),  # two heads per group: 64 tokens per block, beside a decode row
    ],
)
def test_prefill_attention_128_row_blocks_by_size(ops, monkeypatch, hq, hkv, d, lens_new, starts, boost):
    """Steps that reach the 128-row blocks under the host's own rule, nothing forced. Only the last 70
    tokens of the long row and the far key are checked against the slow reference (the whole step would
    take it minutes); the rest against the 64-row blocks, which the cases above pin."""
    seen = spy_prefill_rows(ops, monkeypatch)
    got = attention_tail_case(ops, hq, hkv, d, lens_new, starts, boost, check_last=70)
    assert seen == [128], seen
    monkeypatch.setattr(ops, "PREFILL_BIG_BLOCKS", 1 << 30)
    small = attention_tail_case(ops, hq, hkv, d, lens_new, starts, boost, check_last=0)
    assert seen == [128, 64], seen
    close(got, small, 8e-3, "128-row blocks against 64-row blocks, every token")


def attention_tail_case(ops, hq, hkv, d, lens_new, starts, boost, check_last):
    """As ``attention_case`` in bfloat16 with 16-token pages, but only the last ``check_last`` tokens of row 0 are
    compared with the float64 reference. Returns the kernel's output."""
    page, seed = 16, 50
    g = torch.Generator().manual_seed(seed)
    totals = [s + n for s, n in zip(starts, lens_new)]
    blocks = [-(-tt // page) for tt in totals]
    pages = sum(blocks) + 3
    order = torch.randperm(pages, generator=g).tolist()
    table = torch.full((len(lens_new), max(blocks)), -1, dtype=torch.int32)
    kc, vc = rand((pages, hkv, page, d), BF16, seed + 1), rand((pages, hkv, d, page), BF16, seed + 2)
    at = 0
    for i, nb in enumerate(blocks):
        table[i, :nb] = torch.tensor(order[at : at + nb], dtype=torch.int32)
        at += nb
    t = sum(lens_new)
    q = rand((t, (hq + 2 * hkv) * d), BF16, seed + 3)
    row, where = boost
    last = sum(lens_new[: row + 1]) - 1
    key = kc[table[row, where // page], :, where % page]
    qv = q[last].view(hq + 2 * hkv, d)
    for h in range(hq):
        qv[h] = (key[h // (hq // hkv)].float() * 3.0).to(BF16)
    scale = d**-0.5
    got = ops.paged_attention(q, kc, vc, table.to(DEV), make_batch(lens_new, starts), hq, hkv, d, scale, 0)
    if check_last:
        n0, total = lens_new[0], totals[0]
        idx = table[0].long().to(DEV)
        keys = kc[idx].permute(0, 2, 1, 3).reshape(-1, hkv, d)[:total].double()  # [len, hkv, d]
        vals = vc[idx].permute(0, 3, 1, 2).reshape(-1, hkv, d)[:total].double()
        qd = q.double().view(t, hq + 2 * hkv, d)[:, :hq]
        want = torch.empty((check_last, hq, d), dtype=torch.float64, device=DEV)
        for j in range(check_last):
            tok = n0 - check_last + j
            p = starts[0] + tok
            for h in range(hq):
                kh = h // (hq // hkv)
                wgt = torch.softmax((keys[: p + 1, kh] @ qd[tok, h]) * scale, 0)
                if tok == n0 - 1:
                    assert float(wgt[where]) > 0.9, "the boosted key was meant to dominate"
                want[j, h] = wgt @ vals[: p + 1, kh]
        close(got.view(t, hq, d)[n0 - check_last : n0], want, 8e-3, f"attention {hq}/{hkv}/{d}, the row's last tokens")
    return got


def test_prefill_attention_parts_are_taken(ops, monkeypatch):
    """The cases above do reach the kernel that merges parts: the plan of a short portion far into a
    sequence has parts under the host's own rule, and forcing them changes results by rounding only."""
    assert ops.plan_prefill_parts([64, 1], [6000, 9], 32, 8) is not None
    assert ops.plan_prefill_parts([700], [0], 32, 8) is None
    monkeypatch.setattr(ops, "PREFILL_PARTS_LAUNCH_US", -1e9)
    assert ops.plan_prefill_parts([700], [0], 32, 8) is not None


@pytest.mark.parametrize(
    "hq,hkv,d,starts,window,norm,rot",
    [
        (16, 8, 128, [0, 15, 16, 31, 32, 1000, 4095], 0, True, True),  # page and chunk edges, a sequence of one token
        (16, 8, 128, [700, 3000], 0, False, True),
        (16, 8, 128, [700, 3000, 5], 0, True, False),
        (32, 8, 128, [5, 260, 90], 0, True, True),
        (64, 8, 128, [513, 77], 0, True, True),
        (16, 1, 128, [100, 33], 0, True, True),                        # sixteen query heads on one KV head
        (14, 2, 64, [63, 64, 65, 2000, 1], 0, True, True),             # seven heads per group, head size 64
        (6, 6, 64, [300, 40, 41, 1200], 100, True, True),              # one head per group, a window
        (16, 8, 128, [500, 31, 2047], 33, True, True),
        (4, 2, 128, list(range(0, 6400, 100)), 0, True, True),         # a full batch: one split
        (48, 8, 128, [700, 3000], 0, True, True),                      # three heads per block of the merged projection
        (48, 4, 64, [513, 77, 5], 0, True, True),                      # the same at head size 64, twelve heads per group
        (36, 12, 64, [900, 40], 0, False, True),
        (40, 8, 128, [400, 1300], 0, True, True),                      # 40 heads: no whole number of blocks of three
    ],
)
def test_decode_attention_fused(ops, hq, hkv, d, starts, window, norm, rot):
    """A step of single tokens from the qkv projection's partial sums in one kernel gives what the
    norm / rotation / store kernel followed by the decode attention gives: the outputs, and the new
    token's key and value in the cache. The new token's slots hold NaN beforehand: nothing may be read
    from them."""
    page, eps, b = 16, 1e-6, len(starts)
    g = torch.Generator().manual_seed(5)
    blocks = [-(-(s + 1) // page) for s in starts]
    pages = sum(blocks) + 3
    order = torch.randperm(pages, generator=g).tolist()
    table = torch.full((b, max(blocks)), -1, dtype=torch.int32)
    at = 0
    for i, nb in enumerate(blocks):
        table[i, :nb] = torch.tensor(order[at : at + nb], dtype=torch.int32)
        at += nb
    slots = torch.tensor([int(table[i, s // page]) * page + s % page for i, s in enumerate(starts)], dtype=torch.int32, device=DEV)
    kc, vc = rand((pages, hkv, page, d), BF16, 81), rand((pages, hkv, d, page), BF16, 82)
    x = rand((b, (hq + 2 * hkv) * d), BF16, 83).float()
    parts = torch.stack([x * 0.25, x * 0.5, x * 0.125, x * 0.125, x * 0.0])  # five splits: two rounds of loads
    qw = (rand((d,), BF16, 84) + 1) if norm else None
    kw = (rand((d,), BF16, 85) + 1) if norm else None
    batch = make_batch([1] * b, starts)
    inv_freq = (1.0 / (1e6 ** (torch.arange(0, d, 2).float() / d))).to(DEV)
    rope = ops.rope_table(batch.positions, inv_freq) if rot else None
    scale = d**-0.5
    table = table.to(DEV)
    assert ops.decode_attention_fusable(ops.SplitSum(parts), batch, qw, kw, rope, kc, vc, hq, hkv, d)

    k1, v1 = kc.clone(), vc.clone()
    q = ops.qk_norm_rope_store(ops.SplitSum(parts), slots, qw, kw, eps, rope, k1, v1, hq, hkv, d, out_dtype=BF16)
    want = ops.paged_attention(q, k1, v1, table, batch, hq, hkv, d, scale, window)

    k2, v2 = kc.clone(), vc.clone()
    sl = slots.long()
    k2[sl // page, :, sl % page] = float("nan")
    v2[sl // page, :, :, sl % page] = float("nan")
    assert int(torch.isnan(k2).sum()) == b * hkv * d and int(torch.isnan(v2).sum()) == b * hkv * d
    got = ops.decode_attention_fused(ops.SplitSum(parts), qw, kw, eps, rope, True, k2, v2, table, batch, hq, hkv, d, scale, window)
    close(got, want, 8e-3, f"fused decode attention {hq}/{hkv}/{d}")
    flat = lambda c, v: (c.permute(0, 3, 1, 2) if v else c.permute(0, 2, 1, 3)).reshape(pages * page, hkv, d)
    close(flat(k2, False)[sl], flat(k1, False)[sl], 8e-3, "the new keys in the cache")
    assert torch.equal(flat(v2, True)[sl], flat(v1, True)[sl]), "the new values in the cache"
    rest = torch.ones(pages * page, dtype=torch.bool, device=DEV)
    rest[sl] = False
    assert torch.equal(flat(k2, False)[rest], flat(kc, False)[rest]) and torch.equal(flat(v2, True)[rest], flat(vc, True)[rest])

    # a layer that reads another layer's cache: the new token is in it already, nothing is written
    k3, v3 = k1.clone(), v1.clone()
    got = ops.decode_attention_fused(ops.SplitSum(parts), qw, kw, eps, rope, False, k3, v3, table, batch, hq, hkv, d, scale, window)
    close(got, want, 8e-3, "fused decode attention without the store")
    assert torch.equal(k3, k1) and torch.equal(v3, v1)

    # with the output projection's weight: up to 16 rows whose keys are split come back as the projection's
    # partial sums (the reduction of the splits and the projection are one kernel)
    splits = ops.decode_splits(b, hkv, batch.max_kv_len)
    for n in (192, 4096):  # 64 rows of the weight per block; 256 (a wide weight, many blocks otherwise)
        wo = rand((n, hq * d), BF16, 86, 0.05)
        k4, v4 = kc.clone(), vc.clone()
        got = ops.decode_attention_fused(ops.SplitSum(parts), qw, kw, eps, rope, True, k4, v4, table, batch, hq, hkv, d, scale,
                                         window, project=wo)
        if b <= 16 and 1 < splits <= 64 and hq != 40:
            assert isinstance(got, ops.SplitSum) and got.shape == (b, n) and got.splits <= 16
            close(got.parts.double().sum(0), want.double() @ wo.double().T, 1e-2, f"reduction of the splits and projection in one, {n}")
            assert torch.equal(flat(k4, False)[sl], flat(k2, False)[sl]) and torch.equal(flat(v4, True)[sl], flat(v2, True)[sl])
        else:
            assert isinstance(got, torch.Tensor)
            close(got, want, 8e-3, "no projection where the keys are not split or the rows are many")


def test_decode_splits_rule(ops):
    assert ops.decode_splits(1, 8, 4096) == 32 and ops.decode_splits(8, 8, 4096) == 8 and ops.decode_splits(64, 8, 4096) == 1
    assert ops.decode_splits(1, 8, 100) == 1 and ops.decode_splits(1, 1, 40000) == 312 and ops.decode_splits(1, 8, 1) == 1


def test_attention_one_token_returns_its_value(ops):
    """A sequence of one token: softmax over one key is 1, so the output is v."""
    hq, hkv, d, page = 4, 2, 32, 16
    q = rand((1, (hq + 2 * hkv) * d), F32, 20)
    kc, vc = rand((2, hkv, page, d), F32, 21), rand((2, hkv, d, page), F32, 22)
    table = torch.tensor([[1]], dtype=torch.int32, device=DEV)
    out = ops.paged_attention(q, kc, vc, table, make_batch([1], [0]), hq, hkv, d, d**-0.5, 0).view(hq, d)
    for h in range(hq):
        assert torch.equal(out[h], vc[1, h // 2, :, 0])


def test_attention_refuses_unsupported_head_size(ops):
    q = rand((1, 3 * 24), F32, 23)
    kc, vc = rand((1, 1, 16, 24), F32, 24), rand((1, 1, 24, 16), F32, 24)
    with pytest.raises(ValueError, match="head_dim 24"):
        ops.paged_attention(q, kc, vc, torch.zeros((1, 1), dtype=torch.int32, device=DEV), make_batch([1], [0]), 1, 1, 24, 1.0, 0)


# ------------------------------------------------------------------------------------------ sampling


def test_argmax_takes_the_first_maximum(ops):
    logits = rand((4, 379), F32, 25)
    logits[0, [3, 7]] = 50.0
    logits[3, [30, 5]] = 60.0
    out = ops.sample_rows(logits).cpu().tolist()
    assert out[0] == 3 and out[3] == 5
    assert out[1] == int(logits[1].argmax()) and out[2] == int(logits[2].argmax())


def _as_i32(values):
    return torch.tensor([v - (1 << 32) if v >= (1 << 31) else v for v in values], dtype=torch.int32, device=DEV)


@pytest.mark.parametrize("top_p", [1.0, 0.9, 0.3])
def test_sampling_matches_plain(ops, top_p):
    from plain import qwen3_plain as P

    vocab, rows = 517, 12
    logits = rand((rows, vocab), F32, 26, 3.0)
    temps = [0.0, 0.8, 1.0, 2.0] * 3
    seeds = [1, 2**32 - 1, 12345, 99, 7, 2**31, 0, 5, 6, 7, 8, 9]
    counters = [0, 5, 17, 300, 1, 2, 3, 4, 40, 41, 42, 43]
    got = ops.sample_rows(
        logits, torch.tensor(temps, device=DEV), torch.full((rows,), top_p, device=DEV), _as_i32(seeds),
        torch.tensor(counters, dtype=torch.int32, device=DEV),
    ).cpu().tolist()
    host = logits.cpu().numpy()
    want = [P.sample(host[i], temps[i], seeds[i], counters[i], top_p) for i in range(rows)]
    assert got == want


def test_sampling_frequencies_follow_softmax(ops):
    base = torch.tensor([2, 1, 0.5, 0, -1, -3, 1.5, 0.2], device=DEV)
    n = 50000
    logits = base.repeat(n, 1).contiguous()
    for temp in (0.5, 1.0, 2.0):
        toks = ops.sample_rows(
            logits, torch.full((n,), temp, device=DEV), None, torch.arange(n, dtype=torch.int32, device=DEV),
            torch.zeros(n, dtype=torch.int32, device=DEV),
        )
        freq = torch.bincount(toks.long(), minlength=8).double().cpu() / n
        want = torch.softmax(base.double().cpu() / temp, 0)
        assert float((freq - want).abs().max()) < 0.01


# ------------------------------------------------------------------------------------------ measuring kernels


@pytest.mark.parametrize("vectors,blocks", [(1, 1), (255, 3), (256 * 8 * 5, 4), (256 * 8 * 5 + 77, 4), (100000, 64), (2048 * 9 + 1, 7)])
def test_streaming_read_and_copy_touch_every_vector_once(ops, vectors, blocks):
    """The kernels behind the measured bandwidths: the read's checksums, xor-ed, equal the xor of the
    whole buffer (every 16-byte vector seen exactly once, partial last chunk included), and the copy
    reproduces its source and nothing beyond."""
    g = torch.Generator().manual_seed(vectors)
    src = torch.randint(-(2**31), 2**31 - 1, (vectors * 4,), generator=g, dtype=torch.int64).to(torch.int32).to(DEV)
    sums = ops.measure_read(src, blocks).cpu().numpy().astype(np.uint32)
    want = np.bitwise_xor.reduce(src.cpu().numpy().astype(np.uint32))
    assert np.bitwise_xor.reduce(sums) == want
    dst = torch.full((vectors * 4 + 8,), 7, dtype=torch.int32, device=DEV)
    ops.measure_copy(src, dst[: vectors * 4], blocks)
    assert torch.equal(dst[: vectors * 4], src) and bool((dst[vectors * 4 :] == 7).all())
