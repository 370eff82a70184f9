"""Each HIP kernel alone against a plain float32 reference of the same
operation, at sizes other than the engine's (odd widths, tails of tiles)."""
import math

import numpy as np
import pytest
import torch

import plain_impl
from litinfer_amd.engine.batch import AttentionMeta

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype, f32=1e-5, bf16=2e-2):
    return f32 if dtype is torch.float32 else bf16


def rel(got, ref):
    got = got.double().cpu().numpy() if isinstance(got, torch.Tensor) else got
    return float(np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30))


@pytest.fixture(scope="module")
def ops():
    from litinfer_amd.kernels import ops
    ops.require_gpu(DEV)
    return ops


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(1, 2, 3), (50, 301, 120), (7, 1000, 4096)])
def test_embedding(ops, dtype, shape):
    t, v, h = shape
    g = torch.Generator().manual_seed(0)
    table = torch.randn(v, h, generator=g).to(dtype)
    ids = torch.randint(0, v, (t,), generator=g, dtype=torch.int32)
    out = torch.empty(t, h, device=DEV)
    ops.embedding(ids.to(DEV), table.to(DEV), out)
    ref = plain_impl.embedding(ids.numpy(), table.double().numpy())
    assert np.array_equal(out.double().cpu().numpy(), ref)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape,eps", [((1, 4), 1e-5), ((33, 120), 1e-6), ((512, 4096), 1e-5), ((3, 3584), 1e-6),
                                        ((300, 1002), 1e-6), ((257, 8196), 1e-5), ((256, 20), 0.1)])      # many rows: of any length, too long for registers, short
def test_rmsnorm(ops, dtype, shape, eps):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(*shape, generator=g) * 3
    w = 1 + 0.1 * torch.randn(shape[1], generator=g)
    out = torch.empty(*shape, dtype=dtype, device=DEV)
    ops.rmsnorm(x.to(DEV), w.to(DEV), eps, out)
    ref = plain_impl.rms_norm(x.double().numpy(), w.double().numpy(), eps)
    assert rel(out, ref) < tol(dtype, 2e-6, 8e-3)


def test_rmsnorm_zero_row_is_zero_not_nan(ops):
    x = torch.zeros(2, 64, device=DEV)
    out = torch.empty(2, 64, device=DEV)
    ops.rmsnorm(x, torch.ones(64, device=DEV), 1e-6, out)
    assert torch.equal(out, torch.zeros_like(out))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mnk,bias,acc", [
    ((2, 3, 4), True, False), ((1, 8, 16), False, False), ((5, 301, 120), True, False),
    ((70, 200, 96), False, True), ((130, 129, 264), True, True), ((512, 512, 1024), True, False),
    ((64, 3584, 3584), False, False), ((3, 37, 90), True, False), ((257, 64, 36), False, False),
    ((17, 37, 264), True, True), ((33, 130, 1160), False, False), ((48, 16, 8), True, False),
    ((8, 4608, 3584), True, False), ((65, 50, 128), False, True),
    ((1, 1000, 3584), True, False), ((16, 70, 260), True, True), ((40, 19, 100), False, True),      # few rows in 32-bit
    ((9, 18, 4), True, False),
    ((300, 200, 130), True, True), ((256, 128, 64), False, False), ((1000, 333, 1027), True, False),     # the large 32-bit tile
    ((2048, 3584, 128), True, True), ((2000, 4600, 64), True, False),           # tiles of 256 x 128 and 256 x 256, ragged
    ((1100, 4600, 128), True, True), ((1167, 6627, 128), False, False),         # 192 x 128 and 256 x 192: a last row of tiles with few rows
    ((585, 3979, 128), True, False), ((779, 6296, 128), False, True)])          # four waves one above the other: 128 x 224 and 128 x 288
def test_linear(ops, dtype, mnk, bias, acc):
    m, n, k = mnk
    g = torch.Generator().manual_seed(2)
    x = torch.randn(m, k, generator=g).to(dtype)
    w = (torch.randn(n, k, generator=g) / math.sqrt(k)).to(dtype)
    b = torch.randn(n, generator=g) if bias else None
    ref = plain_impl.linear(x.double().numpy(), w.double().numpy(), None if b is None else b.double().numpy())
    if acc:
        base = torch.randn(m, n, generator=g)
        out = base.to(DEV)
        ref = ref + base.double().numpy()
    else:
        out = torch.empty(m, n, dtype=dtype, device=DEV)
    ops.linear(x.to(DEV), w.to(DEV), None if b is None else b.to(DEV), out, accumulate=acc)
    # operands are exact in both dtypes; what differs is the float32 accumulation over K terms
    # (a random-walk error of about sqrt(K) half-ulps) and, for a bfloat16 out, its rounding
    assert rel(out, ref) < (4 * math.sqrt(k) * 2.0 ** -24 if out.dtype is torch.float32 else 5e-3)


@pytest.mark.parametrize("m,n,k,swiglu,out_dtype,bias,acc", [
    (1, 16, 8, False, torch.bfloat16, False, False),
    (8, 4608, 3584, False, torch.bfloat16, True, False),        # decode: qkv + bias
    (8, 18944, 3584, True, torch.bfloat16, False, False),       # decode: gate/up + swiglu
    (8, 3584, 18944, False, torch.float32, False, True),        # decode: down + residual
    (5, 301, 120, False, torch.float32, False, False),          # odd sizes: head
    (17, 200, 96, True, torch.bfloat16, False, False),
    (32, 37, 264, False, torch.bfloat16, True, False),
    (33, 130, 1160, True, torch.bfloat16, False, False),
    (64, 50, 128, False, torch.float32, True, True),
    (7, 2049, 72, False, torch.float32, True, True),            # few columns: 9 a block, the last block ragged
    (16, 4100, 40, False, torch.bfloat16, True, False),         # 17 a block: two tiles, the second nearly empty
    (12, 8191, 32, False, torch.bfloat16, False, False),        # 32 a block
    (24, 4100, 72, False, torch.float32, True, True),           # the same shares with 17 to 32 rows
    (30, 2500, 40, False, torch.bfloat16, False, False),
    (3, 9000, 64, False, torch.bfloat16, True, False),          # wide output: two tiles a wave
    (16, 8200, 1160, False, torch.float32, True, True),         # wide outputs at other sizes
    (7, 40000, 264, False, torch.float32, False, False),
    (11, 8300, 520, True, torch.bfloat16, False, False),
    (1, 152064, 64, False, torch.float32, False, False),
    (20, 9000, 520, False, torch.bfloat16, False, False),
    (4, 8960, 64, True, torch.bfloat16, False, False),          # gate/up in equal shares of the columns: 12 a block,
    (25, 4101, 40, True, torch.bfloat16, False, False),         # 9 a block with a ragged last one,
    (40, 4864, 72, True, torch.bfloat16, False, False),         # 10 a block
])
def test_linear_skinny_with_fused_swiglu(ops, m, n, k, swiglu, out_dtype, bias, acc):
    g = torch.Generator().manual_seed(12)
    x = (torch.randn(m, k, generator=g) * 2).to(torch.bfloat16)
    w = (torch.randn(2 * n if swiglu else n, k, generator=g) / math.sqrt(k)).to(torch.bfloat16)
    b = torch.randn(n, generator=g) if bias else None
    y = x.double().numpy() @ w.double().numpy().T
    if swiglu:
        y = plain_impl.swiglu(y[:, :n], y[:, n:])
    if b is not None:
        y = y + b.double().numpy()
    if acc:
        base = torch.randn(m, n, generator=g)
        out = base.to(DEV)
        y = y + base.double().numpy()
    else:
        out = torch.full((m, n), float("nan"), dtype=out_dtype, device=DEV)     # a column left out shows
    assert ops.skinny_takes(m, k, w.dtype)
    ops.linear_skinny(x.to(DEV), w.to(DEV), None if b is None else b.to(DEV), out, acc, swiglu=swiglu)
    assert rel(out, y) < (4 * math.sqrt(k) * 2.0 ** -24 if out_dtype is torch.float32 else 5e-3)


class _Lender:
    """Stands in for the engine's workspace."""
    def buffer(self, name, shape, dtype, zero=False):
        return (torch.zeros if zero else torch.empty)(*shape, dtype=dtype, device=DEV)


@pytest.mark.parametrize("m,n,k,out_dtype,bias,acc", [
    (33, 200, 1024, torch.float32, True, True),          # K in parts: few tiles
    (64, 3584, 3584, torch.float32, False, True),
    (48, 300, 18944, torch.bfloat16, True, False),
    (64, 136, 512, torch.bfloat16, False, False),        # too short a K for parts
    (40, 20000, 128, torch.float32, True, False),        # many tiles of 128 columns
    (64, 37000, 64, torch.bfloat16, False, False),       # many tiles of 256 columns
    (128, 3584, 18944, torch.float32, False, True),      # more rows, but few tiles over a long K: parts again
    (200, 300, 4096, torch.bfloat16, True, False),
    (500, 1000, 1024, torch.float32, True, False),       # 32 tiles, two parts
    (13, 3584, 18944, torch.float32, True, True),        # the fewest rows that take the tiles with K in parts (a large matrix)
    (16, 3584, 3584, torch.float32, True, True),         # a small one at 16 rows: the few-row kernel
    (50, 4608, 3584, torch.bfloat16, True, False),       # 36 tiles in 7 parts: not whole eighths, the XCDs share one sequence
    (384, 3584, 2048, torch.float32, False, True),       # 84 tiles in 3 parts, three rows of tiles
    (130, 2048, 1536, torch.float32, True, True),        # 32 tiles in 3 parts: an eighth of the tiles each, part by part
    (64, 1100, 1984, torch.bfloat16, False, False),      # 9 tiles in 3 parts of 11, 10 and 10 steps
])
def test_linear_with_k_in_parts(ops, m, n, k, out_dtype, bias, acc):
    g = torch.Generator().manual_seed(15)
    x = (torch.randn(m, k, generator=g) * 2).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g) / math.sqrt(k)).to(torch.bfloat16)
    b = torch.randn(n, generator=g) if bias else None
    y = x.double().numpy() @ w.double().numpy().T
    if b is not None:
        y = y + b.double().numpy()
    if acc:
        base = torch.randn(m, n, generator=g)
        y = y + base.double().numpy()
    outs = []
    for ws in (_Lender(), None):                         # with and without memory for partial sums
        out = base.to(DEV) if acc else torch.full((m, n), float("nan"), dtype=out_dtype, device=DEV)
        ops.linear(x.to(DEV), w.to(DEV), None if b is None else b.to(DEV), out, acc, ws=ws)
        assert rel(out, y) < (4 * math.sqrt(k) * 2.0 ** -24 if out_dtype is torch.float32 else 5e-3)
        outs.append(out)
    again = base.to(DEV) if acc else torch.empty(m, n, dtype=out_dtype, device=DEV)
    ops.linear(x.to(DEV), w.to(DEV), None if b is None else b.to(DEV), again, acc, ws=_Lender())
    assert torch.equal(again, outs[0])                   # the parts are added in a fixed order


@pytest.mark.parametrize("m,n,k,bias,taken", [
    (64, 3584, 18944, False, True),      # a decoding batch of 64 at the 7B sizes
    (40, 200, 1024, True, True),
    (200, 300, 4096, True, True),        # more than 64 rows, few tiles
    (64, 37000, 64, False, False),       # no cut along K: nothing is done
    (8, 200, 1024, False, False),        # few rows: another kernel's business
    (12, 3584, 18944, False, False),     # the most rows of that kernel's whatever the matrix
    (13, 3584, 3584, True, False),       # 13 to 16 rows against a small matrix: still the few-row kernel
    (13, 3584, 18944, True, True),       # against a large one (136 MB): tiles with K in parts
])
def test_linear_into_the_residual_sum_with_its_norm(ops, m, n, k, bias, taken):
    g = torch.Generator().manual_seed(19)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g) / math.sqrt(k)).to(torch.bfloat16)
    b = torch.randn(n, generator=g) * 0.1 if bias else None
    base = torch.randn(m, n, generator=g) * torch.logspace(-2, 2, m)[:, None]       # rows of very different size
    gamma, eps = torch.rand(n, generator=g) + 0.5, 1e-5
    out = base.to(DEV)
    xn = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    did = ops.linear_then_norm(x.to(DEV), w.to(DEV), None if b is None else b.to(DEV), out, gamma.to(DEV), eps, xn, _Lender())
    assert did == taken
    if not taken:
        assert torch.equal(out.cpu(), base) and torch.isnan(xn.float()).all()        # nothing was touched
        return
    y = base.double().numpy() + x.double().numpy() @ w.double().numpy().T + (0 if b is None else b.double().numpy())
    ref = plain_impl.rms_norm(y, gamma.double().numpy(), eps)
    for i in range(m):
        assert rel(out[i], y[i]) < 4 * math.sqrt(k) * 2.0 ** -24, i
        assert rel(xn[i], ref[i]) < 8e-3, i
    # the sum is the one that the product alone leaves, bit for bit
    alone = base.to(DEV)
    ops.linear(x.to(DEV), w.to(DEV), None if b is None else b.to(DEV), alone, True, ws=_Lender())
    assert torch.equal(alone, out)
    # and the norm is the one that the norm's own kernel makes of that sum, up to the order of its additions
    own = torch.empty_like(xn)
    ops.rmsnorm(out, gamma.to(DEV), eps, own)
    assert (own.float() - xn.float()).abs().max().item() <= 2.0 ** -7 * own.float().abs().max().item()


@pytest.mark.parametrize("m,n,k", [
    (8, 200, 96),                # few rows: the decode kernel
    (13, 9500, 128),             # 13 to 64 rows: tiles of 64 rows
    (40, 20000, 128),
    (64, 9500, 192),
    (50, 18944, 128),            # tiles of 64 x 192: the gates in one wave, the ups in the wave beside it
    (33, 12300, 192),            # the same with a ragged last tile
    (65, 32, 64),                # one tile, one step of K
    (100, 200, 128),             # an output width that is no multiple of 32
    (300, 1000, 192),            # several tiles both ways, ragged edges
    (700, 4700, 256),            # tiles of 256 x 128
    (2048, 18944, 128),          # enough tiles for the largest tiling
    (97, 7419, 128),             # few rows against many columns: tiles of 128 x 192, four waves one above the other
    (300, 9001, 128),            # tiles of 128 x 256
    (1101, 2500, 192),           # nine rows of tiles: the last XCD's share of the tiles is short
    (1024, 4800, 192),           # tiles of 128 x 320: 160 gate columns in one wave, their ups in the wave beside it
    (2000, 4793, 192),           # the same with ragged edges both ways
])
def test_linear_with_swiglu_epilogue(ops, m, n, k):
    g = torch.Generator().manual_seed(14)
    x = (torch.randn(m, k, generator=g) * 2).to(torch.bfloat16)
    w = (torch.randn(2 * n, k, generator=g) / math.sqrt(k)).to(torch.bfloat16)
    y = x.double().numpy() @ w.double().numpy().T
    y = plain_impl.swiglu(y[:, :n], y[:, n:])
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    assert ops.swiglu_takes(m, k, w.dtype)
    ops.linear_swiglu(x.to(DEV), w.to(DEV), out)
    assert rel(out, y) < 5e-3
    # a gate far from zero either way and single outputs that stand out
    w2 = torch.zeros(2 * n, k)
    w2[3, 0] = 30.0; w2[n + 3, 0] = 1.0          # silu(+large) * up
    w2[5, 0] = -30.0; w2[n + 5, 0] = 1.0         # silu(-large) -> 0
    w2[n - 1, 1] = 1.0; w2[2 * n - 1, 1] = 2.0   # the last output
    x2 = torch.zeros(m, k); x2[:, 0] = 1.0; x2[m - 1, 1] = 3.0
    ops.linear_swiglu(x2.to(torch.bfloat16).to(DEV), w2.to(torch.bfloat16).to(DEV), out)
    o = out.float().cpu()
    assert abs(o[0, 3].item() - 30.0) < 0.2 and abs(o[0, 5].item()) < 1e-9
    want_last = 2.0 * 3.0 * (3.0 / (1 + math.exp(-3.0)))
    assert abs(o[m - 1, n - 1].item() - want_last) < 0.1 and o[0, n - 1].item() == 0.0
    assert torch.count_nonzero(o).item() <= 2 * m + 1


@pytest.mark.parametrize("m,inter,k", [(1, 300, 264), (8, 2000, 3584), (16, 37, 100), (17, 4200, 512), (33, 200, 96),
                                       (64, 500, 128), (5, 9000, 1160), (40, 16500, 64)])
def test_float32_few_row_product_with_swiglu_epilogue(ops, m, inter, k):
    """The 32-bit path's gate/up product of a decoding step: on the float32 matrix cores, the activation in
    the epilogue; one, two and four row tiles, one to four column tiles, short and long K."""
    g = torch.Generator().manual_seed(12)
    x = torch.randn(m, k, generator=g)
    w = torch.randn(2 * inter, k, generator=g) / math.sqrt(k)
    y = x.double().numpy() @ w.double().numpy().T
    ref = plain_impl.swiglu(y[:, :inter], y[:, inter:])
    out = torch.full((m, inter), float("nan"), device=DEV)
    assert ops.swiglu_takes(m, k, torch.float32) == (m <= 16)         # (the parts ask; the kernel takes up to 64 rows)
    ops.linear_swiglu(x.to(DEV), w.to(DEV), out)
    assert rel(out, ref) < 8 * math.sqrt(k) * 2.0 ** -24


@pytest.mark.parametrize("m,n,kprev,inter,eps", [
    (8, 3584, 512, 1024, 1e-6),      # a decoding step at the 7B width
    (8, 5120, 256, 27648, 1e-6),     # the 32B's gate/up matrix (566 MB): tiles of 64 x 256 scale the rows
    (3, 3584, 512, 18944, 1e-6),     # the 7B's (272 MB): tiles of 64 x 192
    (16, 5120, 128, 20480, 1e-5),    # 419 MB: tiles of 64 x 192, gates and ups in two waves
    (1, 40, 8, 24, 1e-5),
    (16, 8200, 64, 48, 1e-5),        # a width from which the product before takes 32 columns a block; ragged
    (5, 200, 136, 301, 0.1),         # a ragged last block of 16 columns; an eps that counts
    (9, 264, 72, 8210, 1e-5),        # many outputs, ragged; fewer chunks of K than waves
    (4, 1096, 40, 9000, 1e-6),
    (17, 3584, 512, 1024, 1e-6),     # two tiles of rows a block: the same three ways out, 32 places a block for the shares
    (32, 1536, 8960, 8960, 1e-6),    # the 1.5B's sizes at 32 rows: few-row kernels on both sides
    (24, 3584, 512, 18944, 1e-6),    # the 7B's gate/up at 24 rows: tiles of 64 x 192 scale 24 rows
    (29, 5120, 128, 20480, 1e-5),    # gates and ups in two waves
    (19, 8200, 64, 48, 1e-5),
    (32, 200, 136, 301, 0.1),
    (21, 264, 72, 8210, 1e-5),
])
def test_rms_norm_shared_between_the_products_on_its_two_sides(ops, m, n, kprev, inter, eps):
    """x += h Wo^T leaves gamma * x and the shares of the rows' sums of squares; the gate/up product
    with SwiGLU (and the packed projection with rotary encoding and page write) scales its rows."""
    g = torch.Generator().manual_seed(18)
    h = torch.randn(m, kprev, generator=g).to(torch.bfloat16)
    wo = (torch.randn(n, kprev, generator=g) / math.sqrt(kprev)).to(torch.bfloat16)
    bias = torch.randn(n, generator=g) * 0.1
    base = torch.randn(m, n, generator=g) * torch.logspace(-2, 2, m)[:, None]       # rows of very different size
    gamma = torch.rand(n, generator=g) + 0.5
    x = base.double().numpy() + h.double().numpy() @ wo.double().numpy().T + bias.double().numpy()
    assert ops.residual_norm_takes(m, n, kprev, wo.dtype)
    out = base.to(DEV)
    xg = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    places = ops.row_scale_rows(m)                       # 16 up to 16 rows, 32 above
    parts = torch.full((ops.RESIDUAL_NORM_MAX_PARTS * places,), float("nan"), device=DEV)
    nparts = ops.linear_residual_norm(h.to(DEV), wo.to(DEV), bias.to(DEV), out, gamma.to(DEV), xg, parts)
    assert nparts == ops.residual_norm_parts(n) <= ops.RESIDUAL_NORM_MAX_PARTS
    for i in range(m):
        assert rel(out[i], x[i]) < 1e-5, i
        assert rel(xg[i], gamma.double().numpy() * x[i]) < 2.0 ** -8, i
    sq = parts[:nparts * places].view(nparts, places)[:, :m].double().sum(dim=0).cpu().numpy()
    assert np.allclose(sq, (x * x).sum(axis=1), rtol=1e-5)
    # the same sum as the product alone leaves it
    alone = base.to(DEV)
    ops.linear(h.to(DEV), wo.to(DEV), bias.to(DEV), alone, True)
    assert torch.equal(alone, out)
    scale = ops.RowScale(parts, nparts, eps)
    xn = plain_impl.rms_norm(x, gamma.double().numpy(), eps)
    xb = xg.double().cpu().numpy()                       # what the product after the norm multiplies
    inv = 1.0 / np.sqrt((x * x).mean(axis=1, keepdims=True) + eps)
    # -- gate/up with SwiGLU
    w = (torch.randn(2 * inter, n, generator=g) / math.sqrt(n)).to(torch.bfloat16)
    y = xn @ w.double().numpy().T
    ref = plain_impl.swiglu(y[:, :inter], y[:, inter:])
    got = torch.full((m, inter), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.linear_swiglu(xg, w.to(DEV), got, row_scale=scale)
    yb = (xb @ w.double().numpy().T) * inv
    refb = plain_impl.swiglu(yb[:, :inter], yb[:, inter:])
    for i in range(m):                                   # the kernel's own arithmetic, row by row
        assert rel(got[i], refb[i]) < 5e-3, i
    # against the plain norm and product, element by element within what rounding the rows to
    # bfloat16 (each term by at most 2^-9 of itself) and the output can do:
    # |d out| <= |silu(g)| |d u| + |u| |silu'(g)| |d g| + 2^-9 |out|, |silu'| <= 1.1
    ya = np.abs(xn) @ np.abs(w.double().numpy()).T
    g_, u_ = y[:, :inter], y[:, inter:]
    bound = 2.0 ** -9 * (np.abs(g_ / (1 + np.exp(-g_))) * ya[:, inter:] + 1.1 * np.abs(u_) * ya[:, :inter] + np.abs(ref))
    err = np.abs(got.double().cpu().numpy() - ref)
    assert (err <= 1.01 * bound + 1e-30).all(), float((err / (bound + 1e-30)).max())
    # -- the packed projection with rotary encoding and page write
    nh, nkv, dh, page, pages = 3, 1, 32, 8, 5
    nq = (nh + 2 * nkv) * dh
    wq = (torch.randn(nq, n, generator=g) / math.sqrt(n)).to(torch.bfloat16)
    bq = torch.randn(nq, generator=g)
    pos = torch.randint(0, 3000, (m,), generator=g, dtype=torch.int32)
    slots = torch.randperm(pages * page, generator=g)[:m].to(torch.int32)
    cos = torch.empty(m, dh // 2, device=DEV)
    sin = torch.empty(m, dh // 2, device=DEV)
    ops.rope_table(pos.to(DEV), 1e6, dh, cos, sin)
    kc = torch.zeros((pages, nkv, page, dh), dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros_like(kc)
    q = torch.full((m, nq), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.linear_rope_store(xg, wq.to(DEV), bq.to(DEV), q, nh, nkv, dh, cos, sin, slots.to(DEV), kc, vc, page,
                          row_scale=scale)
    yq = ((xb @ wq.double().numpy().T) * inv + bq.double().numpy()).reshape(m, nh + 2 * nkv, dh)
    refq = np.concatenate([plain_impl.rope_neox(yq[:, :nh + nkv], pos.numpy(), 1e6), yq[:, nh + nkv:]], axis=1)
    assert rel(q, refq.reshape(m, nq)) < 5e-3
    qv = q.cpu().view(m, nh + 2 * nkv, dh)
    for i in range(m):
        sl = int(slots[i])
        assert torch.equal(kc[sl // page, :, sl % page].cpu(), qv[i, nh:nh + nkv])
        assert torch.equal(vc[sl // page, :, sl % page].cpu(), qv[i, nh + nkv:])
    with pytest.raises(ValueError):                      # more rows than the kernels scale
        ops.linear_swiglu(torch.zeros(33, n, dtype=torch.bfloat16, device=DEV), w.to(DEV),
                          torch.empty(33, inter, dtype=torch.bfloat16, device=DEV), row_scale=scale)


@pytest.mark.parametrize("dtype", DTYPES)
def test_linear_rows_do_not_depend_on_the_batch(ops, dtype):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(200, 264, generator=g).to(dtype).to(DEV)
    w = torch.randn(150, 264, generator=g).to(dtype).to(DEV)
    full = torch.empty(200, 150, dtype=torch.float32, device=DEV)
    ops.linear(x, w, None, full)
    for rows in (slice(0, 1), slice(17, 19), slice(100, 200)):
        part = torch.empty(rows.stop - rows.start, 150, dtype=torch.float32, device=DEV)
        ops.linear(x[rows].contiguous(), w, None, part)
        # kernels for few and for many rows may add the K terms in another order: rounding only
        assert rel(part, full[rows].double().cpu().numpy()) < 4 * math.sqrt(264) * 2.0 ** -24


def test_the_rule_for_few_rows_is_the_same_in_the_library_and_in_the_host_stand_in(ops):
    # parts ask the kernel library which kernels few rows should take; the stand-in that the host-side tests
    # run the parts with answers the same
    import torch_ops
    for m in (1, 8, 12, 13, 16, 17, 24, 32, 33, 64, 65):
        for n, k in ((1536, 1536), (3584, 18944), (18944, 3584), (4608, 3584), (5120, 27648), (10240, 8192), (14000, 3745),
                     (17920, 1536), (1536, 8960), (2048, 11008), (5120, 5120), (7168, 5120), (22016, 2048), (300, 100)):
            assert ops.few_rows_preferred(m, n, k) == torch_ops.few_rows_preferred(m, n, k), (m, n, k)
    assert ops.few_rows_preferred(12, 3584, 18944) and not ops.few_rows_preferred(13, 3584, 18944)
    assert ops.few_rows_preferred(16, 3584, 3584) and ops.few_rows_preferred(32, 3584, 3584) and not ops.few_rows_preferred(33, 3584, 3584)
    assert not ops.few_rows_preferred(17, 3584, 18944) and not ops.few_rows_preferred(17, 5120, 5120)
    assert ops.few_rows_preferred(32, 1536, 8960) and not ops.few_rows_preferred(17, 2048, 11008)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(2, 3), (33, 200), (512, 4096)])
def test_swiglu(ops, dtype, shape):
    t, i = shape
    g = torch.Generator().manual_seed(4)
    gu = (torch.randn(t, 2 * i, generator=g) * 3).to(dtype)
    out = torch.empty(t, i, dtype=dtype, device=DEV)
    ops.swiglu(gu.to(DEV), out)
    gd = gu.double().numpy()
    ref = plain_impl.swiglu(gd[:, :i], gd[:, i:])
    assert rel(out, ref) < tol(dtype, 1e-6, 8e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("t,heads,dh,theta,start", [(3, 1, 4, 1e4, 0), (40, 5, 48, 5e4, 7), (64, 4, 128, 1e6, 500)])
def test_rope(ops, dtype, t, heads, dh, theta, start):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(t, heads * dh, generator=g).to(dtype)
    pos = torch.arange(start, start + t, dtype=torch.int32)
    cos = torch.empty(t, dh // 2, device=DEV)
    sin = torch.empty(t, dh // 2, device=DEV)
    ops.rope_table(pos.to(DEV), theta, dh, cos, sin)
    xd = x.to(DEV).clone()
    ops.rope_apply(xd, heads, dh, dh, cos, sin)
    ref = plain_impl.rope_neox(x.double().numpy().reshape(t, heads, dh), pos.numpy(), theta).reshape(t, -1)
    # float32 angles: an angle near `start + t` carries an absolute error of about its ulp
    assert rel(xd, ref) < tol(dtype, 2e-4 if start else 2e-6, 8e-3)


def _paged_case(ops, dtype, seg_specs, nh, nkv, dh, page, window, seed, scale_one=None, row=None, ws=None,
                pad_pow2=False):
    """seg_specs: list of (ctx_len, q_len).  Builds random K/V for every
    segment, scatters them into shuffled pages, and compares the kernel with
    the plain attention on the logical sequences.  `scale_one` is the index of a
    key that is made to stand out for query `row` of its segment (the last one
    when `row` is None).  `pad_pow2`: the block table is widened to the next power
    of two and the decode kernel is told the table's width as its longest context,
    as a recorded decode step sees its batch."""
    g = torch.Generator().manual_seed(seed)
    nseg = len(seg_specs)
    blocks = [-(-c // page) for c, _ in seg_specs]
    num_pages = sum(blocks) + 3
    perm = torch.randperm(num_pages, generator=g).tolist()
    kc = torch.randn(num_pages, nkv, page, dh, generator=g).to(dtype)      # garbage everywhere first
    vc = torch.randn(num_pages, nkv, page, dh, generator=g).to(dtype)
    width = max(blocks) if not pad_pow2 else max(16, 1 << (max(blocks) - 1).bit_length())
    tab = np.full((nseg, width), -1, dtype=np.int32)
    T = sum(q for _, q in seg_specs)
    q = (torch.randn(T, nh * dh, generator=g)).to(dtype)
    ks, vs = [], []
    o = 0
    for s, (c, ql) in enumerate(seg_specs):
        k = torch.randn(c, nkv, dh, generator=g).to(dtype)
        v = torch.randn(c, nkv, dh, generator=g).to(dtype)
        if scale_one is not None:             # make one far key stand out for the last query
            far = scale_one
            big = math.sqrt(12.0 * math.sqrt(dh))      # its score is 12 after scaling: e^12 against some hundred keys near 1
            k[far] = 0
            k[far, :, 0] = big
            r = ql - 1 if row is None else row
            q[o + r].view(nh, dh)[:, :] = 0
            q[o + r].view(nh, dh)[:, 0] = big
        for b in range(blocks[s]):
            tab[s, b] = perm.pop()
            n = min(page, c - b * page)
            kc[tab[s, b], :, :n] = k[b * page:b * page + n].transpose(0, 1)
            vc[tab[s, b], :, :n] = v[b * page:b * page + n].transpose(0, 1)
        ks.append(k)
        vs.append(v)
        o += ql
    q_len = np.array([ql for _, ql in seg_specs], dtype=np.int32)
    ctx_len = np.array([c for c, _ in seg_specs], dtype=np.int32)
    q_start = np.concatenate([[0], np.cumsum(q_len)[:-1]]).astype(np.int32)
    seg_of = np.repeat(np.arange(nseg, dtype=np.int32), q_len)
    dev = lambda a: torch.from_numpy(a).to(DEV)
    single = np.nonzero(q_len[seg_of] == 1)[0].astype(np.int32)
    multi = np.nonzero(q_len[seg_of] != 1)[0].astype(np.int32)
    meta = AttentionMeta(block_table=dev(tab), max_blocks=tab.shape[1], seg_of_token=dev(seg_of),
                         q_start=dev(q_start), q_len=dev(q_len), ctx_len=dev(ctx_len), num_segments=nseg,
                         num_tokens=T, max_q_len=int(q_len.max()), max_ctx_len=int(ctx_len.max()),
                         host_q_start=q_start, host_q_len=q_len, host_ctx_len=ctx_len,
                         single_tokens=dev(single) if len(multi) else None, num_single=len(single),
                         multi_tokens=dev(multi) if len(single) else None, num_multi=len(multi),
                         tiles=dev(np.asarray([(i, int(q_start[i]) + a, min(32, int(q_len[i]) - a), 0)
                                               for i in range(nseg) if q_len[i] > 1
                                               for a in range(0, int(q_len[i]), 32)], dtype=np.int32).reshape(-1, 4)),
                         num_tiles=sum(-(-int(n) // 32) for n in q_len if n > 1), tile_rows=32,
                         max_single_ctx=(width * page if pad_pow2 else int(ctx_len[q_len == 1].max())) if len(single) else 0)
    out = torch.empty(T, nh * dh, dtype=dtype, device=DEV)
    scale = 1.0 / math.sqrt(dh)
    ops.paged_attention(q.to(DEV), out, kc.to(DEV), vc.to(DEV), meta, nh, nkv, dh, page, window, scale, ws=ws)
    refs = []
    o = 0
    for s, (c, ql) in enumerate(seg_specs):
        qq = q[o:o + ql].double().numpy().reshape(ql, nh, dh)
        refs.append(plain_impl.attention(qq, ks[s].double().numpy(), vs[s].double().numpy(),
                                         np.arange(c - ql, c), np.arange(c), scale, window).reshape(ql, -1))
        o += ql
    return out, np.concatenate(refs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("segs,nh,nkv,dh,page,window", [
    ([(2, 2)], 1, 1, 4, 16, 0),                       # the reference's smallest case
    ([(11, 5)], 4, 2, 8, 16, 0),                      # a 5-token portion after 6 cached tokens
    ([(20, 20), (20, 1)], 4, 2, 8, 16, 0),            # shuffled table, last page partly filled
    ([(20, 1), (28, 1)], 4, 2, 8, 16, 0),             # two decoding requests with interleaved pages
    ([(100, 37), (1, 1), (300, 1), (64, 64)], 6, 2, 48, 8, 0),
    ([(100, 37), (33, 2), (300, 1), (70, 70)], 5, 5, 32, 16, 20),    # window crosses pages
    ([(130, 130), (257, 3)], 28, 4, 128, 16, 0),      # the 7B layer's head layout
    ([(200, 8)], 3, 1, 112, 16, 64),
    ([(4096, 1), (37, 1), (1, 1), (700, 1)], 28, 4, 128, 16, 0),    # decoding: keys split over blocks
    ([(900, 1), (64, 1), (2000, 1)], 12, 1, 64, 16, 300),           # 12 heads in one group, window
    ([(1000, 1), (50, 3), (513, 1)], 4, 2, 16, 8, 0),               # decoding beside a portion
    ([(300, 1), (77, 1)], 6, 3, 80, 16, 0),                         # a head size the split kernel does not take
    ([(300, 1), (1025, 1), (31, 1)], 40, 2, 64, 16, 0),             # 20 heads in a group: two blocks of MFMA rows
    ([(33, 1), (32, 1), (1, 1)], 7, 7, 128, 8, 0),                  # one head per group, keys around a block's edge
    ([(700, 700), (40, 3), (513, 1), (300, 17)], 28, 4, 128, 16, 0),    # portions on the matrix cores
    ([(257, 100), (90, 90), (64, 33)], 20, 2, 64, 8, 50),           # 10 heads a group (two turns of waves), window
    ([(2, 2), (17, 16), (33, 2)], 3, 3, 128, 16, 0),
    ([(500, 300), (70, 70), (45, 2)], 8, 2, 128, 12, 0),            # page sizes that do not divide a block of 32 keys
    ([(400, 150), (130, 130)], 6, 3, 128, 64, 90),                  # pages longer than a block of keys, window
    ([(333, 200), (64, 5)], 10, 2, 64, 5, 0),
    ([(300, 300), (100, 9)], 4, 1, 64, 24, 40),
    ([(1, 1), (3000, 700)], 14, 2, 128, 1, 0),                      # one key a page: a long table
    ([(1200, 1200), (40, 3)], 28, 4, 128, 16, 0),                   # more blocks than compute units: the tile's keys in one go
    ([(1300, 1300)], 32, 8, 64, 8, 200),
    ([(5000, 300)], 4, 2, 128, 1, 0),                               # a table too long for the kernel that keeps the pages' offsets in LDS
    ([(1500, 400), (9, 9)], 7, 1, 128, 1, 0),                       # one key a page, within its table
    ([(1100, 1100), (40, 3)], 40, 8, 128, 16, 0),                   # groups of 5 heads: blocks of five waves
    ([(1100, 1100)], 48, 8, 64, 12, 0),                             # groups of 6: six waves, pages that do not divide a block of keys
    ([(2100, 2100)], 18, 2, 64, 8, 700),                            # groups of 9: two blocks of five waves, one of them with four heads
])
def test_paged_attention(ops, dtype, segs, nh, nkv, dh, page, window):
    out, ref = _paged_case(ops, dtype, segs, nh, nkv, dh, page, window, seed=6)
    assert rel(out, ref) < tol(dtype, 3e-6, 1.5e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("far", [3, 1000, 1999])
def test_a_far_key_stands_out_in_a_decode_batch_of_unequal_contexts(ops, far, dtype):
    # contexts of 2,000 to 5,000 keys: the batch gets one run length and a list of its runs; one key of every
    # request (in its first run or a later one) takes nearly all of the weight
    rng = np.random.default_rng(9)
    segs = [(int(c), 1) for c in rng.integers(2000, 5000, 24)] + [(5000, 1), (2000, 1)]
    from litinfer_amd.kernels.ops import _ragged_splits, decode_splits
    class _M: pass
    m = _M()
    m.host_q_len = np.ones(len(segs), dtype=np.int32)
    m.host_ctx_len = np.array([c for c, _ in segs], dtype=np.int32)
    planned = decode_splits(len(segs) * 2, 5000, 1024)
    assert _ragged_splits(planned, m, 0) > planned                 # the case is what it says
    got, ref = _paged_case(ops, dtype, segs, 12, 2, 128, 16, 0, seed=43, scale_one=far, ws=_Lender())
    assert rel(got, ref) < tol(dtype, 1e-5, 8e-3)


@pytest.mark.parametrize("window", [0, 900])
def test_decode_run_length_of_a_batch_with_unequal_contexts(ops, window):
    # the run length chosen on the device against the same search written out, for contexts from 3 to 5,000
    # keys; then the attention of that batch
    rng = np.random.default_rng(5)
    ctx = rng.integers(3, 5000, 37).astype(np.int32)
    ctx[11] = 5000
    nseg, page, nkv, nsplit, simds = len(ctx), 16, 2, 9, 128
    ones = np.ones(nseg, dtype=np.int32)
    dev = lambda a: torch.from_numpy(a).to(DEV)
    max_blocks = 512
    meta = AttentionMeta(block_table=torch.zeros(nseg, max_blocks, dtype=torch.int32, device=DEV), max_blocks=max_blocks,
                         seg_of_token=dev(np.arange(nseg, dtype=np.int32)), q_start=dev(np.arange(nseg, dtype=np.int32)),
                         q_len=dev(ones), ctx_len=dev(ctx), num_segments=nseg, num_tokens=nseg, max_q_len=1,
                         max_ctx_len=int(ctx.max()), host_q_start=np.arange(nseg, dtype=np.int32), host_q_len=ones,
                         host_ctx_len=ctx, num_single=nseg)
    out = torch.full((2 + nseg + nseg * nsplit,), -1, dtype=torch.int32, device=DEV)
    ops.decode_run_keys(meta, None, nseg, page, window, nkv, nsplit, simds, out)
    keys = np.minimum(ctx, window) if window else ctx
    widest = min(max_blocks * page, window) if window else max_blocks * page
    lower, cap = (-(-int(keys.max()) // nsplit) + 31) & ~31, (-(-widest // nsplit) + 31) & ~31
    cost = {c: -(-int(nkv * np.sum(-(-keys // c))) // simds) * (c + 24) for c in range(lower, max(cap, lower) + 1, 32)}
    want = min(cost, key=lambda c: (cost[c], c))
    got = out.cpu().numpy()
    assert int(got[0]) == want
    runs = -(-keys // want)
    assert int(got[1]) == int(runs.sum()) and np.array_equal(got[2:2 + nseg], runs)
    items = got[2 + nseg:2 + nseg + int(runs.sum())]
    assert [(int(i) & 0xffff, int(i) >> 16) for i in items] == [(t, r) for t in range(nseg) for r in range(int(runs[t]))]
    assert want == (832 if not window else 128)      # (without a window the shortest run, 576, is not the cheapest)
    # the same with the runs taken four at a time, as the matrix-core decode kernel's blocks do: a group of
    # fewer runs still holds four SIMDs, and the list names the first run of every group
    nsplit4 = 12
    out = torch.full((2 + nseg + nseg * nsplit4,), -1, dtype=torch.int32, device=DEV)
    ops.decode_run_keys(meta, None, nseg, page, window, nkv, nsplit4, simds, out, group=4)
    lower, cap = (-(-int(keys.max()) // nsplit4) + 31) & ~31, (-(-widest // nsplit4) + 31) & ~31
    cost = {c: -(-int(nkv * np.sum(-(-(-(-keys // c)) // 4) * 4)) // simds) * (c + 24) for c in range(lower, max(cap, lower) + 1, 32)}
    want4 = min(cost, key=lambda c: (cost[c], c))
    got = out.cpu().numpy()
    runs = -(-keys // want4)
    groups = -(-runs // 4)
    assert int(got[0]) == want4 and int(got[1]) == int(groups.sum()) and np.array_equal(got[2:2 + nseg], runs)
    items = got[2 + nseg:2 + nseg + int(groups.sum())]
    assert [(int(i) & 0xffff, int(i) >> 16) for i in items] == [(t, 4 * r) for t in range(nseg) for r in range(int(groups[t]))]
    segs = [(int(c), 1) for c in ctx]
    got, ref = _paged_case(ops, torch.bfloat16, segs, 12, 2, 128, 16, window, seed=41, ws=_Lender())
    assert rel(got, ref) < 8e-3


@pytest.mark.parametrize("segs,nh,nkv,dh,page,window", [
    ([(3000, 64)], 28, 4, 128, 16, 0),                              # two tiles behind 2,936 cached tokens: their keys in five runs
    ([(3000, 64), (500, 1), (1200, 40), (40, 40)], 28, 4, 128, 16, 0),   # beside a decoding token; a short tile leaves runs without keys
    ([(6000, 96)], 12, 2, 64, 8, 3000),                             # a window, six heads a group
    ([(2500, 33), (2600, 2)], 8, 8, 128, 12, 0),                    # pages that do not divide a block of keys; a tile of one row
])
def test_prompt_portions_behind_long_contexts_with_their_keys_in_runs(ops, segs, nh, nkv, dh, page, window):
    from litinfer_amd.kernels.ops import _prefill_runs
    ql, cl = np.array([q for _, q in segs], dtype=np.int32), np.array([c for c, _ in segs], dtype=np.int32)
    blocks = max(-(-c // page) for c, _ in segs)
    assert _prefill_runs(ql, cl, nh, nkv, dh, blocks, window, int(ql.sum())) > 1       # the case is what it says
    out, ref = _paged_case(ops, torch.bfloat16, segs, nh, nkv, dh, page, window, seed=31, ws=_Lender())
    assert rel(out, ref) < 1.5e-2
    # and one far key among thousands, in a run of its own
    for far in (5, 1000, 2900):
        out, ref = _paged_case(ops, torch.bfloat16, [(3000, 64)], 28, 4, 128, 16, 0, seed=32, scale_one=far, row=40, ws=_Lender())
        assert rel(out, ref) < 1.5e-2


# ---- the context lengths of the long workloads (8 x 30,000-token prompts in portions of 2,048, then decoding):
# block tables of 1,875 to 2,048 pages, a portion behind 28,000 cached keys, splits of many pages
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("pad_pow2", [False, True])
@pytest.mark.parametrize("far", [3, 15000, 29940])
def test_decoding_over_thirty_thousand_keys_finds_one_far_key(ops, far, pad_pow2, dtype):
    """Eight requests of 30,000 keys each, pages of 16, 40 heads on 8 kv heads of size 128: one key of every
    request, near the start, in the middle or near the end, carries nearly all the weight.  Also with the
    block table widened to 2,048 pages, as a recorded step sees it."""
    segs = [(30000 - 7 * i, 1) for i in range(8)]
    out, ref = _paged_case(ops, dtype, segs, 40, 8, 128, 16, 0, seed=51, scale_one=far, ws=_Lender(),
                           pad_pow2=pad_pow2)
    assert rel(out, ref) < tol(dtype, 1e-5, 8e-3)


@pytest.mark.parametrize("page,ctx,window", [(1, 5000, 0), (2, 8400, 0), (1, 6000, 4500)])
def test_decode_splits_that_would_hold_more_pages_than_the_kernel_keeps_get_more_runs(ops, page, ctx, window):
    """Many requests with small pages: the number of runs that fills the SIMDs once would give every run
    more than the 1,024 pages the matrix-core decode kernel keeps in LDS, so the host raises the number
    of runs until a run fits; a far key in the first, a middle and the last run."""
    from litinfer_amd.kernels import ops as O
    n, nkv = 64, 4
    segs = [(ctx - 3 * i, 1) for i in range(n)]
    blocks = -(-ctx // page)
    keys = min(ctx, window) if window else ctx
    planned = O.decode_splits(n * nkv, keys, O._simd_count(torch.device(DEV)))
    assert O.decode_split_blocks(blocks, page, window, planned) > O.DECODE_TABLE_CAP      # the case is what it says
    for far in (ctx - 3 * n - 5, ctx // 2, max(ctx - window, 0) + 7 if window else 2):
        out, ref = _paged_case(ops, torch.bfloat16, segs, 8, nkv, 64, page, window, seed=52, scale_one=far, ws=_Lender())
        assert rel(out, ref) < 8e-3
    out, ref = _paged_case(ops, torch.float32, segs, 8, nkv, 64, page, window, seed=52, scale_one=ctx // 2, ws=_Lender())
    assert rel(out, ref) < 1e-5


@pytest.mark.parametrize("far", [5, 14000, 29000])
def test_a_portion_of_2048_behind_28000_cached_keys_finds_one_far_key(ops, far):
    """A prompt portion of 2,048 queries behind 28,000 cached keys (pages of 16: a block table of 1,878
    pages), its tiles' keys cut into runs that are joined afterwards: one key in the first, a middle or
    the last run stands out for one row; all rows against the plain attention."""
    from litinfer_amd.kernels.ops import _prefill_runs
    segs, nh, nkv, dh, page = [(30048, 2048)], 8, 2, 128, 16
    ql, cl = np.array([2048], dtype=np.int32), np.array([30048], dtype=np.int32)
    assert _prefill_runs(ql, cl, nh, nkv, dh, -(-30048 // page), 0, 2048) > 1             # the case is what it says
    out, ref = _paged_case(ops, torch.bfloat16, segs, nh, nkv, dh, page, 0, seed=53, scale_one=far, row=1500, ws=_Lender())
    assert rel(out, ref) < 1.5e-2


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dh", [32, 64, 128])          # 64 and 128 take the matrix-core kernels
def test_paged_attention_finds_one_far_key(ops, dtype, dh):
    # one key among hundreds carries almost all the weight: a kernel that skips
    # or misplaces a page gives a visibly different output
    for far in (0, 15, 16, 333, 511):
        out, ref = _paged_case(ops, dtype, [(512, 1)], 4, 2, dh, 16, 0, seed=7, scale_one=far)
        assert rel(out, ref) < tol(dtype, 3e-6, 1.5e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dh", [32, 64, 128])
@pytest.mark.parametrize("ctx,ql", [(512, 70), (300, 33)])
def test_portions_find_one_far_key_for_any_row_of_a_tile(ops, dtype, dh, ctx, ql):
    # portions: the standout key for the first row of a 32-row tile, its last row, the first
    # row of the next tile and the portion's last row; at the start of the sequence, in the
    # middle, just before the portion and at the row's own position
    for row in (0, 31, 32, ql - 1):
        p = ctx - ql + row
        for far in (0, 97, ctx - ql - 1, p):
            out, ref = _paged_case(ops, dtype, [(ctx, ql)], 6, 2, dh, 16, 0, seed=7, scale_one=far, row=row)
            assert rel(out, ref) < tol(dtype, 3e-6, 1.5e-2), (row, far)
        if p + 1 < ctx:                                # the key after the row's own is not seen
            out, ref = _paged_case(ops, dtype, [(ctx, ql)], 6, 2, dh, 16, 0, seed=7, scale_one=p + 1, row=row)
            assert rel(out, ref) < tol(dtype, 3e-6, 1.5e-2), (row, "next")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dh", [32, 64, 128])
def test_window_edge(ops, dtype, dh):
    # the key just outside the window must not count, the one just inside must
    for window, far, visible in ((32, 512 - 32, True), (32, 512 - 33, False)):
        out, ref = _paged_case(ops, dtype, [(512, 1)], 2, 1, dh, 8, window, seed=8, scale_one=far)
        assert rel(out, ref) < tol(dtype, 3e-6, 1.5e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dh", [32, 64, 128])
@pytest.mark.parametrize("ctx,ql,window", [(512, 70, 48), (300, 33, 100), (512, 70, 37)])
def test_window_edge_for_any_row_of_a_tile(ops, dtype, dh, ctx, ql, window):
    # the first and last row of a 32-row tile, the first row of the next tile, a row whose
    # window begins on a block of 32 keys, and the last row: the key at the window's first
    # position counts, the one before it does not
    rows = {0, 31, 32, ql - 1}
    rows.add(next(r for r in range(ql) if (ctx - ql + r - window + 1) % 32 == 0))
    for row in sorted(rows):
        first = ctx - ql + row - window + 1            # the first key that the row sees
        for far in (first, first - 1):
            assert far >= 0
            out, ref = _paged_case(ops, dtype, [(ctx, ql)], 4, 2, dh, 16, window, seed=8, scale_one=far, row=row)
            assert rel(out, ref) < tol(dtype, 3e-6, 1.5e-2), (row, far - first)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dh,pad", [(48, 5), (48, 16), (128, 0), (20, 0)])      # rows that do and do not start on 16 bytes
def test_rope_kv_store_and_plain_store(ops, dtype, dh, pad):
    g = torch.Generator().manual_seed(9)
    t, nh, nkv, page, pages = 37, 3, 2, 8, 11
    qkv = torch.randn(t, (nh + 2 * nkv) * dh + pad, generator=g).to(dtype)[:, :(nh + 2 * nkv) * dh]
    pos = torch.randint(0, 200, (t,), generator=g, dtype=torch.int32)
    slots = torch.randperm(pages * page, generator=g)[:t].to(torch.int32)
    cos = torch.empty(t, dh // 2, device=DEV)
    sin = torch.empty(t, dh // 2, device=DEV)
    ops.rope_table(pos.to(DEV), 1e4, dh, cos, sin)
    outs = []
    for fused in (True, False):
        d = qkv.to(DEV)
        d = d.clone() if d.is_contiguous() else d      # keep the row stride with its pad
        kc = torch.zeros(pages, nkv, page, dh, dtype=dtype, device=DEV)
        vc = torch.zeros_like(kc)
        if fused:
            ops.rope_kv_store(d, nh, nkv, dh, dh, cos, sin, slots.to(DEV), kc, vc, page)
        else:
            ops.rope_apply(d, nh + nkv, dh, dh, cos, sin)
            ops.kv_store(d, nh, nkv, dh, slots.to(DEV), kc, vc, page)
        outs.append((d[:, :nh * dh].clone(), kc, vc))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    x = qkv.double().numpy()
    kref = plain_impl.rope_neox(x[:, nh * dh:(nh + nkv) * dh].reshape(t, nkv, dh), pos.numpy(), 1e4)
    got = outs[0][1].double().cpu().numpy()
    for i in range(t):
        s = int(slots[i])
        assert np.abs(got[s // page, :, s % page] - kref[i]).max() < tol(dtype, 1e-4, 3e-2)
        assert torch.equal(outs[0][2][s // page, :, s % page].cpu(),
                           qkv[i, (nh + nkv) * dh:].reshape(nkv, dh))


@pytest.mark.parametrize("t,nh,nkv,dh,k,bias", [
    (64, 28, 4, 128, 3584, True),       # a decoding batch of 64 at the 7B layer sizes
    (33, 12, 2, 128, 1536, True),
    (13, 64, 8, 128, 8192, True),       # the fewest rows that are cut along K, against a large matrix (168 MB)
    (40, 6, 2, 64, 1280, False),
    (100, 28, 4, 128, 3584, True),      # more than 64 rows: tiles of 128 rows, K still cut
    (200, 12, 2, 128, 1536, False),
])
def test_projection_cut_along_k_with_rotary_encoding_and_page_write_in_the_adding_up(ops, t, nh, nkv, dh, k, bias):
    g = torch.Generator().manual_seed(31)
    n, page, pages = (nh + 2 * nkv) * dh, 16, max(8, t // 16 + 3)
    x = torch.randn(t, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g) / math.sqrt(k)).to(torch.bfloat16)
    b = torch.randn(n, generator=g) if bias else None
    pos = torch.randint(0, 5000, (t,), generator=g, dtype=torch.int32)
    slots = torch.randperm(pages * page, generator=g)[:t].to(torch.int32)
    cos = torch.empty(t, dh // 2, device=DEV)
    sin = torch.empty(t, dh // 2, device=DEV)
    ops.rope_table(pos.to(DEV), 1e6, dh, cos, sin)
    kc = torch.full((pages, nkv, page, dh), 7.0, dtype=torch.bfloat16, device=DEV)
    vc = torch.full_like(kc, 7.0)
    out = torch.full((t, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    took = ops.linear_rope_store_parts(x.to(DEV), w.to(DEV), None if b is None else b.to(DEV), out, nh, nkv, dh, cos, sin,
                                       slots.to(DEV), kc, vc, page, _Lender())
    assert took
    y = x.double().numpy() @ w.double().numpy().T + (0 if b is None else b.double().numpy())
    y = y.reshape(t, nh + 2 * nkv, dh)
    ref = np.concatenate([plain_impl.rope_neox(y[:, :nh + nkv], pos.numpy(), 1e6), y[:, nh + nkv:]], axis=1).reshape(t, n)
    assert rel(out, ref) < 5e-3
    ov = out.cpu().view(t, nh + 2 * nkv, dh)
    touched = torch.zeros(pages, page, dtype=torch.bool)
    for i in range(t):
        sl = int(slots[i])
        touched[sl // page, sl % page] = True
        assert torch.equal(kc[sl // page, :, sl % page].cpu(), ov[i, nh:nh + nkv])
        assert torch.equal(vc[sl // page, :, sl % page].cpu(), ov[i, nh + nkv:])
    untouched = ~touched[:, None, :, None].expand(pages, nkv, page, dh)
    assert (kc.cpu()[untouched] == 7.0).all() and (vc.cpu()[untouched] == 7.0).all()
    # few rows, or no workspace: not taken
    assert not ops.linear_rope_store_parts(x[:8].to(DEV), w.to(DEV), None, out[:8], nh, nkv, dh, cos[:8], sin[:8],
                                           slots[:8].to(DEV), kc, vc, page, _Lender())


@pytest.mark.parametrize("t,nh,nkv,dh,k,bias", [
    (8, 28, 4, 128, 3584, True),        # a decoding step at the 7B layer sizes
    (1, 3, 1, 32, 96, True),
    (16, 5, 5, 48, 120, False),         # a head size that is no power of two
    (3, 6, 2, 64, 136, True),
    (5, 35, 1, 80, 72, True),           # 1480 rotation pairs: 6 a block, blocks that straddle heads, a ragged last one
    (16, 40, 8, 128, 64, False),        # 3584 pairs: 14 a block, two tiles
    (2, 70, 1, 128, 40, True),          # more pairs than two tiles a compute unit hold: whole tiles again
    (17, 28, 4, 128, 3584, True),       # two tiles of rows a block
    (32, 12, 2, 128, 1536, True),
    (25, 5, 5, 48, 120, False),
    (31, 35, 1, 80, 72, True),
    (20, 70, 1, 128, 40, False),
])
def test_projection_with_rotary_encoding_and_page_write_as_its_epilogue(ops, t, nh, nkv, dh, k, bias):
    g = torch.Generator().manual_seed(16)
    n, page, pages = (nh + 2 * nkv) * dh, 8, 9
    assert t <= page * pages
    x = (torch.randn(t, k, generator=g) * 2).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g) / math.sqrt(k)).to(torch.bfloat16)
    b = torch.randn(n, generator=g) if bias else None
    pos = torch.randint(0, 3000, (t,), generator=g, dtype=torch.int32)
    slots = torch.randperm(pages * page, generator=g)[:t].to(torch.int32)
    cos = torch.empty(t, dh // 2, device=DEV)
    sin = torch.empty(t, dh // 2, device=DEV)
    ops.rope_table(pos.to(DEV), 1e6, dh, cos, sin)
    kc = torch.full((pages, nkv, page, dh), 7.0, dtype=torch.bfloat16, device=DEV)
    vc = torch.full_like(kc, 7.0)
    out = torch.full((t, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    assert ops.rope_store_takes(t, k, w.dtype, dh, dh)
    ops.linear_rope_store(x.to(DEV), w.to(DEV), None if b is None else b.to(DEV), out, nh, nkv, dh, cos, sin,
                          slots.to(DEV), kc, vc, page)
    y = x.double().numpy() @ w.double().numpy().T
    if b is not None:
        y = y + b.double().numpy()
    y = y.reshape(t, nh + 2 * nkv, dh)
    ref = np.concatenate([plain_impl.rope_neox(y[:, :nh + nkv], pos.numpy(), 1e6), y[:, nh + nkv:]], axis=1)
    assert rel(out, ref.reshape(t, n)) < 5e-3
    o = out.cpu().view(t, nh + 2 * nkv, dh)
    touched = torch.zeros(pages, page, dtype=torch.bool)
    for i in range(t):                                   # the pages hold exactly what out holds
        s = int(slots[i])
        touched[s // page, s % page] = True
        assert torch.equal(kc[s // page, :, s % page].cpu(), o[i, nh:nh + nkv])
        assert torch.equal(vc[s // page, :, s % page].cpu(), o[i, nh + nkv:])
    untouched = ~touched[:, None, :, None].expand(pages, nkv, page, dh)
    assert (kc.cpu()[untouched] == 7.0).all() and (vc.cpu()[untouched] == 7.0).all()


@pytest.mark.parametrize("shape", [(1, 4), (3, 4096), (5, 152064), (2, 301)])
def test_argmax_rows_lowest_index_wins(ops, shape):
    g = torch.Generator().manual_seed(10)
    x = torch.randn(*shape, generator=g)
    x[0, shape[1] // 2] = 50.0
    x[0, shape[1] - 1] = 50.0          # an equal maximum later in the row
    out = torch.empty(shape[0], dtype=torch.int32, device=DEV)
    ops.argmax_rows(x.to(DEV), out)
    assert out.cpu().tolist() == [plain_impl.argmax_first(r) for r in x.numpy()]
    assert out[0].item() == shape[1] // 2


def test_gather_and_cast(ops):
    x = torch.randn(10, 37)
    rows = torch.tensor([9, 0, 0, 4], dtype=torch.int32)
    out = torch.empty(4, 37, device=DEV)
    ops.gather_rows(x.to(DEV), rows.to(DEV), out)
    assert torch.equal(out.cpu(), x[rows.long()])
    b = torch.empty(10, 37, dtype=torch.bfloat16, device=DEV)
    ops.cast(x.to(DEV), b)
    assert torch.equal(b.cpu(), x.to(torch.bfloat16))       # round to nearest even, as torch does
    f = torch.empty(10, 37, device=DEV)
    ops.cast(b, f)
    assert torch.equal(f.cpu(), x.to(torch.bfloat16).float())


def _sample(ops, logits, temperature, top_k, top_p, u):
    n = logits.shape[0]
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    f = lambda v, dt: torch.tensor(v, dtype=dt, device=DEV)
    ops.sample_rows(logits.to(DEV), f(temperature, torch.float32), f(top_k, torch.int32),
                    f(top_p, torch.float32), f(u, torch.float32), out)
    return out.cpu().tolist()


def _pick_is_right(row, temperature, top_k, top_p, u, pick, slack=2e-5):
    """The kernel sums in float32 in another order than the plain sampler: the
    pick is right if the uniform number lies within its interval of the CDF,
    give or take the rounding of the sums."""
    ids, p = plain_impl.sampling_candidates(row, temperature, top_k, top_p)
    assert pick in ids.tolist(), f"token {pick} is not among the candidates"
    cum = np.cumsum(p)
    i = ids.tolist().index(pick)
    lo = cum[i - 1] if i else 0.0
    return lo - slack <= u <= cum[i] + slack


@pytest.mark.parametrize("vocab", [8, 301, 4096, 152064])
def test_sample_rows_against_the_plain_sampler(ops, vocab):
    g = torch.Generator().manual_seed(13)
    n = 12
    logits = torch.randn(n, vocab, generator=g) * 3
    logits[1, : min(5, vocab)] = 7.0                       # equal maxima: ties go by index
    temperature = [0.0, 0.7, 1.0, 1.3, 0.8, 1.0, 0.5, 2.0, 1.0, 1.0, 0.9, 1.0]
    top_k = [0, 3, 0, 0, 50, 1, 0, 7, vocab, 0, 5, 2]
    top_p = [1.0, 1.0, 0.9, 0.5, 0.8, 0.3, 1.0, 0.95, 1.0, 0.01, 0.99, 1.0]
    u = torch.rand(n, generator=g).tolist()
    picks = _sample(ops, logits, temperature, top_k, top_p, u)
    rows = logits.double().numpy()
    assert picks[0] == plain_impl.argmax_first(rows[0])                    # temperature 0: greedy
    assert picks[5] == plain_impl.argmax_first(rows[5])                    # top_k 1
    assert picks[9] == plain_impl.argmax_first(rows[9])                    # a tiny top_p keeps the maximum only
    for r in range(1, n):
        assert _pick_is_right(rows[r], temperature[r], top_k[r], top_p[r], u[r], picks[r]), r
    # exact agreement wherever the uniform number is not at an interval's edge
    same = sum(picks[r] == plain_impl.sample_with_uniform(rows[r], temperature[r], top_k[r], top_p[r], u[r])
               for r in range(n))
    assert same >= n - 1


@pytest.mark.parametrize("vocab", [8, 301, 8192, 8193, 152064])
def test_sample_rows_with_temperature_alone(ops, vocab):
    # no top-k and no top-p: the kernel's short way; uniform numbers at both ends among them
    g = torch.Generator().manual_seed(15)
    n = 24
    logits = torch.randn(n, vocab, generator=g) * 4
    temperature = [0.3 + 0.1 * i for i in range(n)]
    u = torch.rand(n, generator=g).tolist()
    u[0], u[1], u[2] = 0.0, 0.99999994, 0.5
    picks = _sample(ops, logits, temperature, [0] * n, [1.0] * n, u)
    rows = logits.double().numpy()
    for r in range(n):
        assert 0 <= picks[r] < vocab
        assert _pick_is_right(rows[r], temperature[r], 0, 1.0, u[r], picks[r]), r
    # and mostly the very id of the float64 sampler (among 152,064 ids a float32 sum's rounding moves an
    # interval's edge past the uniform number now and then; each such pick was checked above)
    same = sum(picks[r] == plain_impl.sample_with_uniform(rows[r], temperature[r], 0, 1.0, u[r]) for r in range(n))
    assert same >= n - 4


def test_sample_rows_with_tiles_of_the_vocabulary_masked_out(ops):
    # the rows' ids are summed in tiles of 8,192 first: a tile of -inf alone, a tile so far below the
    # maximum that it has no mass in float32, and the last tile cut short must not disturb the pick
    g = torch.Generator().manual_seed(16)
    vocab, n = 3 * 8192 + 5, 16
    logits = torch.randn(n, vocab, generator=g) * 2
    logits[:8, 8192:16384] = float("-inf")
    logits[8:12, :8192] -= 200.0
    logits[12:, 16384:] = float("-inf")                      # the last two tiles, the short one among them
    temperature = [0.0, 1.0, 0.7, 1.5] * 4
    u = torch.rand(n, generator=g).tolist()
    u[1], u[2], u[5], u[13] = 0.99999994, 0.0, 0.99999994, 0.99999994
    picks = _sample(ops, logits, temperature, [0] * n, [1.0] * n, u)
    rows = logits.double().numpy()
    for r in range(n):
        assert np.isfinite(rows[r][picks[r]]), r
        if temperature[r] == 0.0:
            assert picks[r] == plain_impl.argmax_first(rows[r])
        else:
            assert _pick_is_right(rows[r], temperature[r], 0, 1.0, u[r], picks[r]), r
    assert all(p < 8192 or p >= 16384 for p in picks[:8]) and all(p >= 8192 for p in picks[9:12]) and all(p < 16384 for p in picks[12:])


@pytest.mark.parametrize("vocab", [1000, 20000, 152064])
def test_sample_rows_with_many_equal_logits_at_the_thresholds(ops, vocab):
    # logits on a coarse grid: hundreds of ids share the k-th largest value and the value at which top-p
    # cuts, spread over the threads and tiles of the kernel; which of them survive goes by ascending id
    g = torch.Generator().manual_seed(17)
    n = 16
    logits = torch.round(torch.randn(n, vocab, generator=g) * 2) / 2
    temperature = [1.0, 0.5, 2.0, 0.8] * 4
    top_k = [50, 0, 300, 7, 1000, 0, 2, 64, 999, 0, 50, 50, 0, 5000, 20, 1][:n]
    top_k = [min(k, vocab - 1) for k in top_k]
    top_p = [1.0, 0.6, 0.9, 0.5, 0.95, 0.99, 1.0, 0.3, 1.0, 0.05, 0.8, 0.999, 0.9, 0.7, 1.0, 1.0]
    u = torch.rand(n, generator=g).tolist()
    u[0], u[1], u[2] = 0.99999994, 0.0, 0.99999994
    picks = _sample(ops, logits, temperature, top_k, top_p, u)
    rows = logits.double().numpy()
    for r in range(n):
        assert _pick_is_right(rows[r], temperature[r], top_k[r], top_p[r], u[r], picks[r]), r
    same = sum(picks[r] == plain_impl.sample_with_uniform(rows[r], temperature[r], top_k[r], top_p[r], u[r]) for r in range(n))
    assert same >= n - 2


def test_sample_rows_frequencies_and_ties(ops):
    lg = torch.tensor([[2.0, 1.0, 3.0, 3.0, -1.0, 0.5, 2.5, 0.0]])
    n = 4000
    g = torch.Generator().manual_seed(14)
    u = torch.rand(n, generator=g).tolist()
    picks = _sample(ops, lg.repeat(n, 1), [1.0] * n, [0] * n, [1.0] * n, u)
    freq = np.bincount(picks, minlength=8) / n
    want = np.exp(lg[0].double().numpy())
    assert np.abs(freq - want / want.sum()).max() < 0.03
    # top_k = 1 with two equal maxima: the lower index; top_k = 3: ids 2, 3 and 6 only
    assert set(_sample(ops, lg.repeat(50, 1), [1.0] * 50, [1] * 50, [1.0] * 50, u[:50])) == {2}
    assert set(_sample(ops, lg.repeat(500, 1), [1.0] * 500, [3] * 500, [1.0] * 500, u[:500])) == {2, 3, 6}
    # top_p = 0.5: the shortest prefix reaching half the mass is {2, 3}
    assert set(_sample(ops, lg.repeat(500, 1), [1.0] * 500, [0] * 500, [0.5] * 500, u[:500])) == {2, 3}


def test_sampling_table_rows_become_the_arrays_of_a_step_with_uniform_numbers_drawn_on_the_device(ops):
    """li_sample_prepare against the host's stream: the same uniform numbers bit for bit for any seed and
    count, a count that goes up for sampling rows only, greedy flags, slots outside the table."""
    from litinfer_amd.sampling import Sampler, SamplingParams, uniform
    smp = Sampler(DEV, slots=6)
    opts = [SamplingParams(temperature=0.8, top_k=7, top_p=0.9, seed=0), SamplingParams(temperature=1.5, seed=2 ** 64 - 1),
            SamplingParams(), SamplingParams(temperature=0.3, top_p=0.5, seed=-12345678901234),
            SamplingParams(temperature=1.0, seed=0x9E3779B97F4A7C15)]
    draws = [0, 5, 0, 2 ** 31 - 3, 1000000]
    for slot, (sp, c) in enumerate(zip(opts, draws)):
        smp.bind(slot, sp, c)
    rows = torch.tensor([4, 0, 3 | ops.SAMPLE_ROW_GREEDY, 2, 1, 5, 77], dtype=torch.int32, device=DEV)
    n = rows.numel()
    t, p, u = (torch.full((n,), -1.0, device=DEV) for _ in range(3))
    k = torch.full((n,), -1, dtype=torch.int32, device=DEV)
    for step in range(3):
        ops.sample_prepare(rows, smp.table, t, k, p, u)
        for i, slot in enumerate((4, 0, None, 2, 1, None, None)):      # None: greedy by flag, an unbound row, outside the table
            if slot is None or opts[slot].greedy:
                assert float(t[i]) == 0.0 and float(u[i]) == 0.0
                continue
            sp = opts[slot]
            assert float(t[i]) == np.float32(sp.temperature) and int(k[i]) == sp.top_k and float(p[i]) == np.float32(sp.top_p)
            assert float(u[i]) == uniform(sp.seed, draws[slot] + step), (slot, step)
    counts = smp.table[:, 5].cpu().tolist()
    assert counts == [3, 8, 0, draws[3], 1000003, 0]               # slot 3 was greedy by flag: its count stayed


def test_decode_attention_refuses_block_tables_beyond_the_keys_its_page_quotient_is_exact_for(ops):
    """The matrix-core decode kernel finds a key's page by a float32 product that is exact below 2^22; the host
    refuses a table that could hold more than 2^21 keys instead of reading a wrong page."""
    nh, nkv, dh, page = 4, 2, 128, 16
    width = (1 << 21) // page + 1
    tab = torch.zeros(1, width, dtype=torch.int32, device=DEV)
    one = lambda v: torch.tensor([v], dtype=torch.int32, device=DEV)
    ql, cl, qs = np.array([1], np.int32), np.array([40], np.int32), np.array([0], np.int32)
    meta = AttentionMeta(block_table=tab, max_blocks=width, seg_of_token=one(0), q_start=one(0), q_len=one(1),
                         ctx_len=one(40), num_segments=1, num_tokens=1, max_q_len=1, max_ctx_len=40, host_q_start=qs,
                         host_q_len=ql, host_ctx_len=cl, single_tokens=None, num_single=1, multi_tokens=None,
                         num_multi=0, max_single_ctx=40)
    kc = torch.zeros(4, nkv, page, dh, dtype=torch.bfloat16, device=DEV)
    q = torch.zeros(1, nh * dh, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError, match="beyond the decode kernel"):
        ops.paged_attention(q, torch.empty_like(q), kc, kc.clone(), meta, nh, nkv, dh, page, 0, 0.1)
