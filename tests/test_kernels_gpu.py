"""Each HIP kernel alone against its plain reference (`torch_kernels.TorchKernels`, float32 torch arithmetic),
at sizes other than the engine's: widths and vocabularies that are no power of two, head sizes 16..256, one and
several kv heads, page sizes 4..32."""

import math
from types import SimpleNamespace

import pytest
import torch

from torch_kernels import TorchKernels, philox_first

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def hip():
    """The kernel set as the engine builds it: the BLAS library takes bfloat16 products of more than 16 rows."""
    from ampere_kv_engine_amd.kernels.hip import HipKernels
    return HipKernels("cuda:0")


@pytest.fixture(scope="module")
def hip_own():
    """Every product in the engine's own kernels, whatever the number of rows."""
    from ampere_kv_engine_amd.kernels.hip import HipKernels
    return HipKernels("cuda:0", library_products_above=None)


@pytest.fixture(scope="module")
def hip_library():
    """Every bfloat16 product of more than 16 rows in the BLAS library (a table of choices that names it for all)."""
    from ampere_kv_engine_amd.kernels.hip import HipKernels

    class Always(dict):
        def get(self, key, default=None):
            return "library"
    kernels = HipKernels("cuda:0")
    kernels.product_choices = Always()
    return kernels


@pytest.fixture(params=["own", "library"])
def hip_either(request, hip_own, hip_library):
    return {"own": hip_own, "library": hip_library}[request.param]


@pytest.fixture(scope="module")
def ref():
    return TorchKernels()


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-6) if dtype == torch.float32 else dict(rtol=1.6e-2, atol=1e-3)


def assert_close_but_for_flipped_roundings(got, want):
    """A product whose rows were normed with the squares added in another order: a normed value on a rounding
    boundary now and then falls to the other side (one bfloat16 step of a value of size ~1 to 4), which moves a whole
    output row by that step times a weight.  So: nearly all outputs within the usual limit, none further off than a
    small part of the largest output."""
    got, want = got.float().cpu(), want.float().cpu()
    t = tol(torch.bfloat16)
    outside = (got - want).abs() > t["atol"] + t["rtol"] * want.abs()
    assert outside.float().mean() < 1e-3, f"{int(outside.sum())} of {outside.numel()} outside the usual limit"
    beyond = ((got - want).abs() - t["rtol"] * want.abs()).clamp(min=0).max()
    assert beyond <= 2.0 ** -9 * want.abs().max(), "an output is off by more than a flipped rounding explains"


def attention_tol(dtype):
    """bfloat16: the reference's own bound for its paged attention against float32 attention
    (ampere_kv/scheduler.py:410, ampere_kv/paged_decode.py:62-81: rtol 0.01, atol 0.002); softmax weights enter the
    weighted sum rounded to bfloat16, which alone moves an output by up to ~2^-9 of the values' size."""
    return dict(rtol=2e-5, atol=2e-6) if dtype == torch.float32 else dict(rtol=0.01, atol=0.002)


def rand(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed(hip, ref, dtype):
    table = rand(379, 96, dtype=dtype, seed=1)
    ids = torch.tensor([0, 378, 5, 5, 17], dtype=torch.int32)
    want = torch.empty(5, 96)
    ref.embed(ids, table, want)
    got = torch.empty(5, 96, device="cuda")
    hip.embed(ids.cuda(), table.cuda(), got)
    torch.testing.assert_close(got.cpu(), want, rtol=0, atol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [96, 1000, 4096, 5120, 8192, 10240, 16388, 18000])
def test_add_rmsnorm(hip, ref, dtype, hidden):
    stream = rand(7, hidden, seed=2, scale=3.0)
    delta = rand(7, hidden, dtype=dtype, seed=3)
    weight = 1 + rand(hidden, seed=4, scale=0.1)
    for d in (delta, None):
        s_ref, s_hip = stream.clone(), stream.clone().cuda()
        want = torch.empty(7, hidden, dtype=dtype)
        ref.add_rmsnorm(s_ref, d, weight, 1e-5, want)
        got = torch.empty(7, hidden, dtype=dtype, device="cuda")
        hip.add_rmsnorm(s_hip, d.cuda() if d is not None else None, weight.cuda(), 1e-5, got)
        torch.testing.assert_close(s_hip.cpu(), s_ref, rtol=0, atol=0)          # the residual sum itself
        torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_heads_and_copy(hip, ref, dtype):
    tokens, heads, width = 5, 3, 48
    wide = rand(tokens, 7 * width, dtype=dtype, seed=5)
    view = wide[:, 2 * width:5 * width].unflatten(1, (heads, width))           # a strided view, as inside qkv
    weight = 1 + rand(width, seed=6, scale=0.1)
    want = torch.empty(tokens, heads, width, dtype=dtype)
    ref.rmsnorm_heads(view, weight, 1e-6, want)
    got = torch.empty(tokens, heads, width, dtype=dtype, device="cuda")
    hip.rmsnorm_heads(wide.cuda()[:, 2 * width:5 * width].unflatten(1, (heads, width)), weight.cuda(), 1e-6, got)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dtype))
    copied = torch.empty(tokens, heads, width, dtype=dtype, device="cuda")
    hip.copy_heads(wide.cuda()[:, 2 * width:5 * width].unflatten(1, (heads, width)), copied)
    torch.testing.assert_close(copied.cpu(), view.contiguous(), rtol=0, atol=0)
    flat = rand(11, 200, dtype=dtype, seed=7)
    w2 = 1 + rand(200, seed=8, scale=0.1)
    want2 = torch.empty_like(flat)
    ref.rmsnorm(flat, w2, 1e-5, want2)
    got2 = torch.empty(11, 200, dtype=dtype, device="cuda")
    hip.rmsnorm(flat.cuda(), w2.cuda(), 1e-5, got2)
    torch.testing.assert_close(got2.cpu().float(), want2.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_gather_rows(hip, ref, dtype):
    stream, pending = rand(9, 96, seed=9), rand(9, 96, dtype=dtype, seed=10)
    rows = torch.tensor([8, 0, 3, 3], dtype=torch.int32)
    for p in (pending, None):
        want = torch.empty(4, 96)
        ref.gather_rows(stream, p, rows, want)
        got = torch.empty(4, 96, device="cuda")
        hip.gather_rows(stream.cuda(), p.cuda() if p is not None else None, rows.cuda(), got)
        torch.testing.assert_close(got.cpu(), want, rtol=0, atol=0)


@pytest.mark.parametrize("x_dtype,w_dtype,y_dtype", [
    (torch.float32, torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16, torch.bfloat16),
    (torch.bfloat16, torch.bfloat16, torch.float32), (torch.float32, torch.bfloat16, torch.float32),
    (torch.bfloat16, torch.float32, torch.bfloat16)])
@pytest.mark.parametrize("rows,outs,k", [(1, 379, 96), (5, 64, 200), (70, 130, 33), (129, 257, 1000)])
def test_linear(hip, ref, x_dtype, w_dtype, y_dtype, rows, outs, k):
    x, w = rand(rows, k, dtype=x_dtype, seed=11), rand(outs, k, dtype=w_dtype, seed=12, scale=0.05)
    want = torch.empty(rows, outs, dtype=y_dtype)
    ref.linear(x, w, want)
    got = torch.empty(rows, outs, dtype=y_dtype, device="cuda")
    hip.linear(x.cuda(), w.cuda(), got)
    t = dict(rtol=1e-4, atol=1e-5) if y_dtype == torch.float32 else tol(torch.bfloat16)
    torch.testing.assert_close(got.cpu().float(), want.float(), **t)


@pytest.mark.parametrize("y_dtype", DTYPES)
@pytest.mark.parametrize("rows", [1, 5, 16, 17, 33, 64, 65, 130, 300])
@pytest.mark.parametrize("outs,k", [(379, 96), (64, 4096), (200, 200), (8192, 256), (1040, 1000)])
def test_linear_packed(hip_either, ref, y_dtype, rows, outs, k):
    hip = hip_either
    """bfloat16 weights packed for the matrix cores: few rows (k split over waves), many rows (LDS-staged tiles),
    sizes that are no multiple of the 16 x 32 tile."""
    from ampere_kv_engine_amd.kernels.hip import PackedWeight
    x = rand(rows, k, dtype=torch.bfloat16, seed=31)
    w = rand(outs, k, dtype=torch.bfloat16, seed=32, scale=0.05)
    packed = hip.prepare_linear(w.cuda())
    assert isinstance(packed, PackedWeight) and torch.equal(packed.unpack().cpu(), w)
    want = torch.empty(rows, outs, dtype=y_dtype)
    ref.linear(x, w, want)
    got = torch.full((rows, outs), float("nan"), dtype=y_dtype, device="cuda")
    hip.linear(x.cuda(), packed, got)
    t = dict(rtol=2e-4, atol=2e-5 * k ** 0.5) if y_dtype == torch.float32 else tol(torch.bfloat16)
    torch.testing.assert_close(got.cpu().float(), want.float(), **t)


@pytest.mark.parametrize("outs,k", [(379, 96), (4096, 4096), (1040, 1000), (5136, 2048)])
def test_products_with_a_bias(hip_either, ref, outs, k, monkeypatch):
    """y = x W^T + b with the bias added to the float32 sums before they are rounded (one rounding, as
    torch.nn.functional.linear makes it), through every kernel a product can take: the plain float32 kernel; the
    engine's own kernels at 1 to 64 rows, the mid-size one, the library or the wide one beyond; the decode products
    that add themselves to the residual sum, norm their rows (one and two row tiles a wave) or norm their single
    row.  The bias is large beside the products, so a kernel that drops it, or adds it to the wrong feature, fails."""
    hip = hip_either
    monkeypatch.setattr(hip, "fold_norms", True)
    monkeypatch.setattr(hip, "FOLD_NORM_ROWS", 16)
    w = rand(outs, k, dtype=torch.bfloat16, seed=36, scale=0.05)
    bias = rand(outs, dtype=torch.bfloat16, seed=37, scale=0.7).float()     # (as read from a 16-bit file: exact in bfloat16)
    packed = hip.prepare_linear(w.cuda())
    for rows in (1, 9, 16, 17, 40, 64, 100, 200, 300, 600):
        x = rand(rows, k, dtype=torch.bfloat16, seed=38)
        for y_dtype in DTYPES:
            want = torch.empty(rows, outs, dtype=y_dtype)
            ref.linear(x, w, want, bias)
            got = torch.full((rows, outs), float("nan"), dtype=y_dtype, device="cuda")
            hip.linear(x.cuda(), packed, got, bias=bias.cuda())
            t = dict(rtol=2e-4, atol=2e-5 * k ** 0.5) if y_dtype == torch.float32 else tol(torch.bfloat16)
            torch.testing.assert_close(got.cpu().float(), want.float(), **t, msg=lambda m: f"{rows} rows into {y_dtype}: {m}")
    # the plain kernel, float32 throughout
    x32, w32 = rand(70, k, seed=39), w.float()
    want = torch.empty(70, outs)
    ref.linear(x32, w32, want, bias)
    got = torch.empty(70, outs, device="cuda")
    hip.linear(x32.cuda(), w32.cuda(), got, bias=bias.cuda())
    torch.testing.assert_close(got.cpu(), want, rtol=1e-4, atol=1e-6 * k ** 0.5)     # (sums of k float32 products)
    # the decode products
    for rows in (1, 5, 16):
        x = rand(rows, k, dtype=torch.bfloat16, seed=40)
        stream = rand(rows, outs, seed=41, scale=2.0)
        y = torch.empty(rows, outs, dtype=torch.bfloat16)
        ref.linear(x, w, y, bias)
        residual, sums = stream.cuda(), torch.full(((outs + 15) // 16, 16), float("nan"), device="cuda")
        hip.linear_adds(x.cuda(), packed, residual, sums, bias=bias.cuda())
        torch.testing.assert_close(residual.cpu(), stream + y.float(), rtol=0, atol=2.0 ** -7 * y.float().abs().max().item())
        torch.testing.assert_close(sums.cpu().sum(0)[:rows].double(), residual.cpu().double().pow(2).sum(-1), rtol=1e-5, atol=1e-6)
        if rows * k * 2 > hip.FOLD_NORM_BYTES:
            continue
        rows_in = rand(rows, k, seed=42, scale=2.0)
        gain = 1 + rand(k, seed=43, scale=0.1)
        squares = torch.zeros((k + 15) // 16, 16)
        padded = torch.zeros(rows, squares.shape[0] * 16)
        padded[:, :k] = rows_in
        squares[:, :rows] = (padded * padded).view(rows, -1, 16).sum(-1).T
        normed, want = torch.empty(rows, k, dtype=torch.bfloat16), torch.empty(rows, outs, dtype=torch.bfloat16)
        ref.add_rmsnorm(rows_in.clone(), None, gain, 1e-6, normed)
        ref.linear(normed, w, want, bias)
        for row_tiles in (0, 1, 2):
            got = torch.full((rows, outs), float("nan"), dtype=torch.bfloat16, device="cuda")
            hip.linear_scaled(rows_in.cuda(), squares.cuda(), gain.cuda(), 1e-6, packed, got, row_tiles=row_tiles, bias=bias.cuda())
            assert_close_but_for_flipped_roundings(got, want)
        if rows == 1 and k * 2 <= 48 * 1024:
            new = torch.empty(rows, k, device="cuda")
            got = torch.full((rows, outs), float("nan"), dtype=torch.bfloat16, device="cuda")
            hip.linear_after_norm(rows_in.cuda(), None, gain.cuda(), 1e-6, new, packed, got, bias=bias.cuda())
            assert_close_but_for_flipped_roundings(got, want)
    assert int(hip._exchange_arrivals.abs().sum()) == 0


def test_linear_packed_rows_do_not_depend_on_the_batch(hip_own, monkeypatch):
    hip = hip_own
    """A row's result is bit-identical alone and among up to 64 rows in the skinny kernel, and among more in the wide
    one (the mid-size kernel, which would take these by default, cuts k by the number of rows: its rows agree within
    rounding only - see test_mid_size_product)."""
    for bucket in (2, 3, 4, 8, 16, 32):
        monkeypatch.setitem(hip.product_choices, ("linear", 300, 512, bucket), "own")
    x = rand(200, 512, dtype=torch.bfloat16, seed=33).cuda()
    packed = hip.prepare_linear(rand(300, 512, dtype=torch.bfloat16, seed=34).cuda())
    for count in (40, 200):
        whole = torch.empty(count, 300, device="cuda")
        hip.linear(x[:count].contiguous(), packed, whole)
        for first, n in ((0, 1), (17, 3), (39, 1)) if count == 40 else ((0, 70), (100, 100)):
            part = torch.empty(n, 300, device="cuda")
            hip.linear(x[first:first + n].contiguous(), packed, part)
            assert torch.equal(part, whole[first:first + n])


@pytest.mark.parametrize("y_dtype", DTYPES)
@pytest.mark.parametrize("rows", [1, 7, 16, 17, 40, 64, 65, 128, 300])
@pytest.mark.parametrize("inter,k", [(16, 96), (48, 4096), (208, 200), (4112, 256), (1040, 1000)])
def test_gated_linear(hip_either, ref, y_dtype, rows, inter, k):
    hip = hip_either
    """silu(x Wg^T) * (x Wu^T) in one pass over gate and up tiles that alternate in the packing: numbers of tiles
    that fill no wave's or block's share, few rows and many."""
    from ampere_kv_engine_amd.kernels.hip import GatedWeight
    x = rand(rows, k, dtype=torch.bfloat16, seed=35)
    gate = rand(inter, k, dtype=torch.bfloat16, seed=36, scale=0.08)
    up = rand(inter, k, dtype=torch.bfloat16, seed=37, scale=0.05)
    weight = hip.prepare_gated_linear(gate.cuda(), up.cuda())
    assert isinstance(weight, GatedWeight)
    back = weight.unpack()
    assert torch.equal(back[0].cpu(), gate) and torch.equal(back[1].cpu(), up)
    want = torch.empty(rows, inter, dtype=y_dtype)
    ref.gated_linear(x, (gate, up), want)
    got = torch.full((rows, inter), float("nan"), dtype=y_dtype, device="cuda")
    shape = hip.gated_scratch(weight, rows, y_dtype)
    library = hip.library_products_above is not None and rows > 16 and y_dtype == torch.bfloat16
    assert (shape is not None) == (library and hip._route("gated", inter, k, rows, True, y_dtype) == "library")
    hip.gated_linear(x.cuda(), weight, got, torch.empty(shape, dtype=y_dtype, device="cuda") if shape else None)
    t = dict(rtol=2e-4, atol=2e-5 * k ** 0.5) if y_dtype == torch.float32 else tol(torch.bfloat16)
    torch.testing.assert_close(got.cpu().float(), want.float(), **t)


def test_gated_linear_rows_do_not_depend_on_the_batch_and_other_sizes_stay_stacked(hip_own, monkeypatch):
    hip = hip_own
    for bucket in (2, 3, 4, 8, 16, 32):
        monkeypatch.setitem(hip.product_choices, ("gated", 304, 512, bucket), "own")
    x = rand(200, 512, dtype=torch.bfloat16, seed=38).cuda()
    weight = hip.prepare_gated_linear(rand(304, 512, dtype=torch.bfloat16, seed=39).cuda(),
                                      rand(304, 512, dtype=torch.bfloat16, seed=40).cuda())
    for count in (40, 200):
        whole = torch.empty(count, 304, device="cuda")
        hip.gated_linear(x[:count].contiguous(), weight, whole)
        for first, n in ((0, 1), (17, 3), (39, 1)) if count == 40 else ((0, 70), (100, 100)):
            part = torch.empty(n, 304, device="cuda")
            hip.gated_linear(x[first:first + n].contiguous(), weight, part)
            assert torch.equal(part, whole[first:first + n])
    assert hip.prepare_gated_linear(torch.zeros(40, 64, dtype=torch.bfloat16), torch.zeros(40, 64, dtype=torch.bfloat16)) is None
    assert hip.prepare_gated_linear(torch.zeros(48, 64), torch.zeros(48, 64)) is None


@pytest.mark.parametrize("rows", [1, 3, 4])
@pytest.mark.parametrize("outs,k", [(320, 256), (6144, 4096), (48, 520), (4096, 5120)])
@pytest.mark.parametrize("with_delta", [True, False])
def test_linear_after_norm(hip, ref, rows, outs, k, with_delta):
    """The product whose blocks norm the rows themselves against the norm kernel followed by the product; the new
    residual sum goes to the other buffer, the old one stays."""
    stream = rand(rows, k, seed=61, scale=2.0)
    delta = rand(rows, k, dtype=torch.bfloat16, seed=62) if with_delta else None
    gain = 1 + rand(k, seed=63, scale=0.1)
    w = rand(outs, k, dtype=torch.bfloat16, seed=64, scale=0.05)
    want_stream, normed = stream.clone(), torch.empty(rows, k, dtype=torch.bfloat16)
    ref.add_rmsnorm(want_stream, delta, gain, 1e-5, normed)
    want = torch.empty(rows, outs, dtype=torch.bfloat16)
    ref.linear(normed, w, want)
    packed = hip.prepare_linear(w.cuda())
    assert hip.norm_in_product(1, packed, torch.bfloat16) and not hip.norm_in_product(2, packed, torch.bfloat16)
    old, new = stream.cuda(), torch.full((rows, k), float("nan"), device="cuda")
    got = torch.full((rows, outs), float("nan"), dtype=torch.bfloat16, device="cuda")
    hip.NORM_IN_PRODUCT_ROWS = 4         # what the kernel takes; the engine uses it for one row
    try:
        hip.linear_after_norm(old, delta.cuda() if with_delta else None, gain.cuda(), 1e-5, new, packed, got)
    finally:
        del hip.NORM_IN_PRODUCT_ROWS
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(torch.bfloat16))
    torch.testing.assert_close(new.cpu(), want_stream, rtol=0, atol=0)
    torch.testing.assert_close(old.cpu(), stream, rtol=0, atol=0)


@pytest.mark.parametrize("rows", [1, 4])
def test_gated_linear_after_norm(hip, ref, rows):
    inter, k = 208, 264
    stream = rand(rows, k, seed=65, scale=2.0)
    delta = rand(rows, k, dtype=torch.bfloat16, seed=66)
    gain = 1 + rand(k, seed=67, scale=0.1)
    gate, up = (rand(inter, k, dtype=torch.bfloat16, seed=68 + i, scale=0.05) for i in range(2))
    want_stream, normed = stream.clone(), torch.empty(rows, k, dtype=torch.bfloat16)
    ref.add_rmsnorm(want_stream, delta, gain, 1e-6, normed)
    want = torch.empty(rows, inter, dtype=torch.bfloat16)
    ref.gated_linear(normed, ref.prepare_gated_linear(gate, up), want)
    weight = hip.prepare_gated_linear(gate.cuda(), up.cuda())
    new = torch.empty(rows, k, device="cuda")
    got = torch.full((rows, inter), float("nan"), dtype=torch.bfloat16, device="cuda")
    hip.NORM_IN_PRODUCT_ROWS = 4
    try:
        hip.linear_after_norm(stream.cuda(), delta.cuda(), gain.cuda(), 1e-6, new, weight, got)
    finally:
        del hip.NORM_IN_PRODUCT_ROWS
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(torch.bfloat16))
    torch.testing.assert_close(new.cpu(), want_stream, rtol=0, atol=0)


@pytest.mark.parametrize("rows", [1, 3, 8, 16])
@pytest.mark.parametrize("outs,k", [(320, 256), (4096, 4096), (520, 48), (4096, 12288), (1000, 1032), (5120, 3416)])
def test_a_product_adds_itself_to_the_residual_sum_and_leaves_its_rows_sums_of_squares(hip, ref, rows, outs, k, monkeypatch):
    """`linear_adds` against the product followed by the sum: the new residual rows are the same bits (the product is
    rounded to bfloat16 before it is added, as a stored one would be), and the partial sums add up to the rows' sums of
    squares.  Widths that are no multiple of 16 or 32, a k that is cut over the waves of a block, and one that is not."""
    monkeypatch.setattr(hip, "fold_norms", True)
    monkeypatch.setattr(hip, "FOLD_NORM_ROWS", 16)       # what the kernels take; the engine folds steps of fewer rows
    stream = rand(rows, outs, seed=71, scale=2.0)
    x = rand(rows, k, dtype=torch.bfloat16, seed=72)
    w = rand(outs, k, dtype=torch.bfloat16, seed=73, scale=0.05)
    y = torch.empty(rows, outs, dtype=torch.bfloat16)
    ref.linear(x, w, y)
    packed = hip.prepare_linear(w.cuda())
    # (any 16 rows; with `fold_rows_left` off the engine folds only where the next product, which then norms the rows
    # itself, can hold them in LDS)
    assert hip.adds_to_stream(rows, packed, torch.bfloat16)
    monkeypatch.setattr(hip, "fold_rows_left", False)
    assert hip.adds_to_stream(rows, packed, torch.bfloat16) == (rows * outs * 2 <= hip.FOLD_NORM_BYTES)
    monkeypatch.setattr(hip, "fold_rows_left", True)
    assert not hip.adds_to_stream(17, packed, torch.bfloat16)
    got = stream.cuda()
    tiles = (outs + 15) // 16
    sums = torch.full((tiles, 16), float("nan"), device="cuda")
    hip.linear_adds(x.cuda(), packed, got, sums)
    mine = torch.empty(rows, outs, dtype=torch.bfloat16, device="cuda")
    hip.linear(x.cuda(), packed, mine)          # the same tiles, maybe another cut of k: a last bit here and there
    apart = (got.cpu() - (stream + mine.cpu().float())).abs()
    assert (apart > 0).float().mean() < 0.01 and apart.max() <= 2.0 ** -7 * mine.float().abs().max().item()
    torch.testing.assert_close(got.cpu(), stream + y.float(), rtol=0, atol=2.0 ** -7 * y.float().abs().max().item())
    sums = sums.cpu()
    assert torch.isfinite(sums).all() and (sums[:, rows:] == 0).all()
    padded = torch.zeros(rows, tiles * 16)
    padded[:, :outs] = got.cpu()
    want_sums = padded.double().pow(2).reshape(rows, tiles, 16).sum(-1).T
    torch.testing.assert_close(sums[:, :rows].double(), want_sums, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("rows,outs,k", [(1, 320, 256), (16, 320, 256), (2, 6144, 4096), (8, 6144, 4096), (5, 48, 520),
                                         (16, 48, 520), (6, 4096, 5120), (1, 1000, 1032), (13, 1000, 1032),
                                         (11, 256, 96), (10, 400, 96), (16, 12288, 4096), (3, 512, 10240), (7, 512, 10240)])
def test_a_product_norms_its_rows_from_the_sums_of_squares_it_is_given(hip, ref, rows, outs, k, monkeypatch):
    """`linear_scaled` against the norm kernel followed by the product.  The sums it is given are those of another
    product's `linear_adds`, so the pair is what a layer runs; the residual rows are left as they are."""
    monkeypatch.setattr(hip, "fold_norms", True)
    monkeypatch.setattr(hip, "FOLD_NORM_ROWS", 16)       # what the kernels take; the engine folds steps of fewer rows
    stream = rand(rows, k, seed=74, scale=2.0)
    x = rand(rows, 64, dtype=torch.bfloat16, seed=75)
    before = rand(k, 64, dtype=torch.bfloat16, seed=76, scale=0.2)
    gain = 1 + rand(k, seed=77, scale=0.1)
    w = rand(outs, k, dtype=torch.bfloat16, seed=78, scale=0.05)
    residual = stream.cuda()
    sums = torch.full(((k + 15) // 16, 16), float("nan"), device="cuda")
    hip.linear_adds(x.cuda(), hip.prepare_linear(before.cuda()), residual, sums)
    rows_now = residual.cpu()
    normed, want = torch.empty(rows, k, dtype=torch.bfloat16), torch.empty(rows, outs, dtype=torch.bfloat16)
    ref.add_rmsnorm(rows_now.clone(), None, gain, 1e-5, normed)
    ref.linear(normed, w, want)
    packed = hip.prepare_linear(w.cuda())
    assert hip.norms_rows_in_product(rows, packed, torch.bfloat16)
    assert not hip.norms_rows_in_product(hip.FOLD_NORM_BYTES // (2 * k) + 1, packed, torch.bfloat16)     # the rows must fit into LDS
    got = torch.full((rows, outs), float("nan"), dtype=torch.bfloat16, device="cuda")
    hip.linear_scaled(residual, sums, gain.cuda(), 1e-5, packed, got)
    assert_close_but_for_flipped_roundings(got, want)
    torch.testing.assert_close(residual.cpu(), rows_now, rtol=0, atol=0)
    # against this kernel set's own norm and product the difference is a last bit of a normed value here and there
    mine_normed = torch.empty(rows, k, dtype=torch.bfloat16, device="cuda")
    hip.add_rmsnorm(residual.clone(), None, gain.cuda(), 1e-5, mine_normed)
    mine = torch.empty(rows, outs, dtype=torch.bfloat16, device="cuda")
    hip.linear(mine_normed, packed, mine)
    assert (got.float() - mine.float()).abs().max() <= 0.02 * mine.float().abs().max()
    assert (got != mine).float().mean() < 0.05


@pytest.mark.parametrize("rows,inter,k", [(1, 208, 264), (16, 208, 264), (7, 12288, 4096), (8, 1008, 520), (16, 1008, 520)])
def test_a_gated_product_norms_its_rows_from_the_sums_of_squares(hip, ref, rows, inter, k, monkeypatch):
    monkeypatch.setattr(hip, "fold_norms", True)
    monkeypatch.setattr(hip, "FOLD_NORM_ROWS", 16)       # what the kernels take; the engine folds steps of fewer rows
    inter = (inter + 15) // 16 * 16
    residual = rand(rows, k, seed=79, scale=2.0).cuda()
    gain = 1 + rand(k, seed=80, scale=0.1)
    gate, up = (rand(inter, k, dtype=torch.bfloat16, seed=81 + i, scale=0.05) for i in range(2))
    padded = torch.zeros(rows, (k + 15) // 16 * 16)
    padded[:, :k] = residual.cpu()
    sums = torch.zeros((k + 15) // 16, 16)
    sums[:, :rows] = padded.pow(2).reshape(rows, -1, 16).sum(-1).T
    normed, want = torch.empty(rows, k, dtype=torch.bfloat16), torch.empty(rows, inter, dtype=torch.bfloat16)
    ref.add_rmsnorm(residual.cpu().clone(), None, gain, 1e-6, normed)
    ref.gated_linear(normed, ref.prepare_gated_linear(gate, up), want)
    weight = hip.prepare_gated_linear(gate.cuda(), up.cuda())
    assert hip.norms_rows_in_product(rows, weight, torch.bfloat16)
    got = torch.full((rows, inter), float("nan"), dtype=torch.bfloat16, device="cuda")
    hip.linear_scaled(residual, sums.cuda(), gain.cuda(), 1e-6, weight, got)
    assert_close_but_for_flipped_roundings(got, want)


@pytest.mark.parametrize("rows", [1, 8, 16])
@pytest.mark.parametrize("outs,k", [(5120, 8192), (5120, 5120), (5136, 8200), (5120, 17416)])
def test_row_tiles_whose_parts_of_k_lie_in_two_blocks(hip, ref, rows, outs, k, monkeypatch):
    """The decode products cut their work into equal blocks even where that splits a row tile's parts of k between two
    blocks (320 row tiles on 256 compute units); the two exchange their sums through memory and the later one finishes
    the tile.  Against the same products made to keep whole row tiles in a block (no exchange memory): equal up to the
    order of the sum; twice in a row, since the counters must be back at zero; and against the double."""
    monkeypatch.setattr(hip, "fold_norms", True)
    monkeypatch.setattr(hip, "FOLD_NORM_ROWS", 16)
    x = rand(rows, k, dtype=torch.bfloat16, seed=91)
    w = rand(outs, k, dtype=torch.bfloat16, seed=92, scale=0.05)
    packed = hip.prepare_linear(w.cuda())
    plan = hip.decode_plan(packed)
    assert plan["straddles"] and plan["blocks"] <= 256 and plan["waves"] % plan["k_split"] != 0, plan
    stream = rand(rows, outs, seed=93, scale=2.0)
    want = torch.empty(rows, outs, dtype=torch.bfloat16)
    ref.linear(x, w, want)
    tiles = (outs + 15) // 16

    def adds():
        got, sums = stream.cuda(), torch.full((tiles, 16), float("nan"), device="cuda")
        hip.linear_adds(x.cuda(), packed, got, sums)
        return got.cpu(), sums.cpu()

    first, second = adds(), adds()
    assert torch.equal(first[0], second[0]) and torch.equal(first[1], second[1])
    assert int(hip._exchange_arrivals.abs().sum()) == 0
    with monkeypatch.context() as patch:
        patch.setattr(hip, "_exchange", lambda n_tiles: (None, None))
        whole = adds()
    apart = (first[0] - whole[0]).abs()
    assert (apart > 0).float().mean() < 0.01 and apart.max() <= 2.0 ** -7 * want.float().abs().max().item()
    torch.testing.assert_close(first[0], stream + want.float(), rtol=0, atol=2.0 ** -7 * want.float().abs().max().item())
    torch.testing.assert_close(first[1].sum(0)[:rows].double(), first[0].double().pow(2).sum(-1), rtol=1e-5, atol=1e-6)
    # the product that norms its rows, over the same matrix read the other way round (k of the norm = outs here)
    if rows * outs * 2 <= hip.FOLD_NORM_BYTES and outs % 8 == 0:
        back = hip.prepare_linear(rand(5120, outs, dtype=torch.bfloat16, seed=94, scale=0.05).cuda())
        gain = 1 + rand(outs, seed=95, scale=0.1)
        residual, sums = first[0].cuda(), first[1].cuda()

        def scaled():
            got = torch.full((rows, 5120), float("nan"), dtype=torch.bfloat16, device="cuda")
            hip.linear_scaled(residual, sums, gain.cuda(), 1e-6, back, got)
            return got.cpu()

        got = scaled()
        assert torch.equal(got, scaled()) and int(hip._exchange_arrivals.abs().sum()) == 0
        normed, want_back = torch.empty(rows, outs, dtype=torch.bfloat16), torch.empty(rows, 5120, dtype=torch.bfloat16)
        ref.add_rmsnorm(first[0].clone(), None, gain, 1e-6, normed)
        ref.linear(normed, back.unpack().cpu(), want_back)
        assert_close_but_for_flipped_roundings(got, want_back)


@pytest.mark.parametrize("rows", [3, 16])
@pytest.mark.parametrize("outs", [8208, 10256, 10272])      # 513, 641 and 642 row tiles: odd and even numbers of them
def test_pairs_of_row_tiles_whose_parts_of_k_lie_in_two_blocks(hip, ref, rows, outs, monkeypatch):
    """The product that norms its rows, with two row tiles a wave (forced: the sizes alone never choose it where
    blocks share wave-rows) and so many row tiles that the blocks do not hold whole wave-rows: the exchange memory is
    indexed by wave-row and holds two tiles for each - with an odd number of row tiles the last wave-row reaches one
    tile beyond the matrix.  Against one row tile a wave (same sums, other order) and the double; twice, for the
    counters; and nothing beyond the exchange memory's own end is touched."""
    monkeypatch.setattr(hip, "fold_norms", True)
    monkeypatch.setattr(hip, "FOLD_NORM_ROWS", 16)
    k = 2048
    w = rand(outs, k, dtype=torch.bfloat16, seed=61, scale=0.05)
    packed = hip.prepare_linear(w.cuda())
    plan = hip.decode_plan(packed, row_tiles_per_wave=2, normed_rows=rows)
    assert plan["straddles"], plan
    assert hip._exchange_tiles >= packed.n_tiles + 1
    stream = rand(rows, k, seed=62, scale=2.0)
    gain = 1 + rand(k, seed=63, scale=0.1)
    sums = torch.zeros((k + 15) // 16, 16)
    sums[:, :rows] = (stream * stream).view(rows, -1, 16).sum(-1).T
    normed, want = torch.empty(rows, k, dtype=torch.bfloat16), torch.empty(rows, outs, dtype=torch.bfloat16)
    ref.add_rmsnorm(stream.clone(), None, gain, 1e-6, normed)
    ref.linear(normed, w, want)
    guard = hip._exchange_pieces[(packed.n_tiles + 1) * 512:(packed.n_tiles + 1) * 512 + 4096]
    guard.fill_(-77.0)

    def scaled(row_tiles):
        got = torch.full((rows, outs), float("nan"), dtype=torch.bfloat16, device="cuda")
        hip.linear_scaled(stream.cuda(), sums.cuda(), gain.cuda(), 1e-6, packed, got, row_tiles=row_tiles)
        return got.cpu()

    pairs = scaled(2)
    assert torch.equal(pairs, scaled(2)) and int(hip._exchange_arrivals.abs().sum()) == 0
    assert bool((guard == -77.0).all()), "the exchange wrote beyond the tiles it was given"
    assert_close_but_for_flipped_roundings(pairs, want)
    assert_close_but_for_flipped_roundings(pairs, scaled(1))


def test_exchanging_products_give_the_same_bits_two_hundred_times(hip, hip_own, monkeypatch):
    """Products whose blocks hand sums to each other through memory (decode products whose row tiles straddle blocks;
    mid-size products whose k is cut over blocks) are called 200 times back to back, each call on a copy of the matrix
    that no cache holds, with other kernels' reads in between: every result equals the first bit for bit (the parts are
    added in a fixed order whoever arrives last), and the counters are back at zero.  Stops at the first mismatch."""
    monkeypatch.setattr(hip, "fold_norms", True)
    monkeypatch.setattr(hip, "FOLD_NORM_ROWS", 16)
    spacer = torch.zeros(96 << 20, dtype=torch.float32, device="cuda")       # 384 MB: more than the caches hold
    cases = []
    # decode: o and down at sizes whose 320 row tiles meet 256 compute units; the product that norms its rows likewise
    for rows, outs, k in ((8, 5120, 8192), (16, 5120, 5120), (1, 5120, 17416)):
        x = rand(rows, k, dtype=torch.bfloat16, seed=71).cuda()
        copies = [hip.prepare_linear(rand(outs, k, dtype=torch.bfloat16, seed=72, scale=0.05).cuda()) for _ in range(3)]
        assert hip.decode_plan(copies[0])["straddles"]
        base = rand(rows, outs, seed=73, scale=2.0).cuda()

        def adds(i, x=x, copies=copies, base=base, rows=rows, outs=outs):
            stream, sums = base.clone(), torch.empty((outs + 15) // 16, 16, device="cuda")
            hip.linear_adds(x, copies[i % 3], stream, sums)
            return torch.cat((stream.view(-1), sums.view(-1)))
        cases.append((f"adds {rows} x {outs} x {k}", adds))
        if rows * outs * 2 <= hip.FOLD_NORM_BYTES:
            back = [hip.prepare_linear(rand(5120, outs, dtype=torch.bfloat16, seed=74, scale=0.05).cuda()) for _ in range(3)]
            sums = torch.rand((outs + 15) // 16, 16, device="cuda")
            gain = (1 + rand(outs, seed=75, scale=0.1)).cuda()

            def scaled(i, base=base, sums=sums, gain=gain, back=back, rows=rows):
                out = torch.empty(rows, 5120, dtype=torch.bfloat16, device="cuda")
                hip.linear_scaled(base, sums, gain, 1e-6, back[i % 3], out)
                return out.view(-1).float()
            cases.append((f"scaled {rows} x 5120 x {outs}", scaled))
    # mid-size: the four products of a layer at 128 and 40 rows (their cuts divide k over blocks)
    import ctypes
    for rows in (128, 40):
        for outs, k in ((6144, 4096), (4096, 4096), (4096, 12288)):
            x = rand(rows, k, dtype=torch.bfloat16, seed=76).cuda()
            copies = [hip_own.prepare_linear(rand(outs, k, dtype=torch.bfloat16, seed=77, scale=0.05).cuda()) for _ in range(3)]
            need, words = ctypes.c_long(0), ctypes.c_long(0)
            hip_own.lib.akv_linear_mid_workspace(rows, copies[0].n_tiles, copies[0].k_tiles, 0, 0, 0, 0, 0, ctypes.byref(need), ctypes.byref(words))
            assert need.value > 0, "this product's k is not cut over blocks"

            def mid(i, x=x, copies=copies, rows=rows, outs=outs):
                out = torch.empty(rows, outs, dtype=torch.float32, device="cuda")
                hip_own._mid(x, copies[i % 3], out, rows, outs, False)
                return out.view(-1)
            cases.append((f"mid {rows} x {outs} x {k}", mid))
    for name, call in cases:
        first = call(0).clone()
        for turn in range(1, 201):      # (the copies hold the same values: every call must equal the first)
            if turn % 2:
                spacer.sum()            # other work between the calls, and the caches emptied
            got = call(turn)
            assert torch.equal(got, first), f"{name}: call {turn} differs from the first in {int((got != first).sum())} values"
    assert int(hip._exchange_arrivals.abs().sum()) == 0 and int(hip_own._mid_counters.abs().sum()) == 0


def test_decode_products_at_random_sizes(hip, ref, monkeypatch):
    """The products that add themselves to the residual sum and norm their rows, at sixty random sizes - outputs and k
    that are no multiples of the tiles, every number of rows, small matrices (one block) and large ones (blocks that
    share row tiles) - against the double's product, sum and norm."""
    monkeypatch.setattr(hip, "fold_norms", True)
    monkeypatch.setattr(hip, "FOLD_NORM_ROWS", 16)
    generator = torch.Generator().manual_seed(2024)
    pick = lambda low, high: int(torch.randint(low, high + 1, (1,), generator=generator))
    for case in range(60):
        large = case % 6 == 0
        rows = pick(1, 16)
        outs = pick(4800, 7200) if large else pick(1, 700)
        k = 8 * (pick(500, 1100) if large else pick(1, 300))
        hidden = 8 * pick(2, 300)                      # width of the residual rows that the second product norms
        x = rand(rows, k, dtype=torch.bfloat16, seed=1000 + case)
        w = rand(hidden, k, dtype=torch.bfloat16, seed=2000 + case, scale=0.05)
        stream = rand(rows, hidden, seed=3000 + case, scale=2.0)
        what = f"case {case}: rows {rows}, {hidden} x {k}, then {outs} x {hidden}"
        y = torch.empty(rows, hidden, dtype=torch.bfloat16)
        ref.linear(x, w, y)
        residual = stream.cuda()
        tiles = (hidden + 15) // 16
        sums = torch.full((tiles, 16), float("nan"), device="cuda")
        hip.linear_adds(x.cuda(), hip.prepare_linear(w.cuda()), residual, sums)
        scale = y.float().abs().max().item()
        torch.testing.assert_close(residual.cpu(), stream + y.float(), rtol=0, atol=2.0 ** -7 * scale, msg=lambda m: f"{what}: {m}")
        torch.testing.assert_close(sums.cpu().sum(0)[:rows].double(), residual.cpu().double().pow(2).sum(-1), rtol=1e-5, atol=1e-6,
                                   msg=lambda m: f"{what}: {m}")
        assert (sums.cpu()[:, rows:] == 0).all(), what
        if rows * hidden * 2 > hip.FOLD_NORM_BYTES:
            continue
        gain = 1 + rand(hidden, seed=4000 + case, scale=0.1)
        second = rand(outs, hidden, dtype=torch.bfloat16, seed=5000 + case, scale=0.05)
        normed, want = torch.empty(rows, hidden, dtype=torch.bfloat16), torch.empty(rows, outs, dtype=torch.bfloat16)
        ref.add_rmsnorm(residual.cpu().clone(), None, gain, 1e-6, normed)
        ref.linear(normed, second, want)
        got = torch.full((rows, outs), float("nan"), dtype=torch.bfloat16, device="cuda")
        hip.linear_scaled(residual, sums, gain.cuda(), 1e-6, hip.prepare_linear(second.cuda()), got)
        assert torch.isfinite(got.float()).all(), what
        assert_close_but_for_flipped_roundings(got, want)
    assert int(hip._exchange_arrivals.abs().sum()) == 0


def test_products_of_17_to_512_rows_follow_a_table_that_is_measured_on_request(hip, ref, tmp_path):
    """Which kernel takes a product of 17..512 rows - the skinny one (up to 64), the mid-size one, the library - is
    decided by a fixed rule unless the table of choices names the product (matrix shape and row bucket).  Nothing is
    timed by a product call; `measure_products` fills the table for the shapes prepared so far and reports every
    decision; the table can be saved and loaded; every choice gives the product."""
    from ampere_kv_engine_amd.kernels.hip import HipKernels
    kernels = HipKernels("cuda:0")
    w = rand(320, 256, dtype=torch.bfloat16, seed=41, scale=0.05)
    packed = kernels.prepare_linear(w.cuda())
    gate, up = (rand(64, 256, dtype=torch.bfloat16, seed=43 + i, scale=0.05) for i in range(2))
    gated = kernels.prepare_gated_linear(gate.cuda(), up.cuda())

    def products():
        for rows in (8, 20, 31, 64, 65, 130, 300, 600):
            x = rand(rows, 256, dtype=torch.bfloat16, seed=42)
            want = torch.empty(rows, 320, dtype=torch.bfloat16)
            ref.linear(x, w, want)
            got = torch.full((rows, 320), float("nan"), dtype=torch.bfloat16, device="cuda")
            kernels.linear(x.cuda(), packed, got)
            torch.testing.assert_close(got.cpu().float(), want.float(), **tol(torch.bfloat16))
            want = torch.empty(rows, 64, dtype=torch.bfloat16)
            ref.gated_linear(x, ref.prepare_gated_linear(gate, up), want)
            got = torch.full((rows, 64), float("nan"), dtype=torch.bfloat16, device="cuda")
            shape = kernels.gated_scratch(gated, rows, torch.bfloat16)
            scratch = torch.empty(shape, dtype=torch.bfloat16, device="cuda") if shape is not None else None
            kernels.gated_linear(x.cuda(), gated, got, scratch)
            torch.testing.assert_close(got.cpu().float(), want.float(), **tol(torch.bfloat16))
    products()
    assert kernels.product_choices == {}                       # calls decide nothing
    lines = []
    table = kernels.measure_products(log=lines.append)
    assert set(table) == {(kind, outs, 256, bucket) for kind, outs in (("linear", 320), ("gated", 64))
                          for bucket in (2, 3, 4, 8, 16, 32)}
    assert set(table.values()) <= {"own", "mid", "library"} and len(lines) == 12 and all("->" in line for line in lines)
    products()
    for forced in ("own", "mid", "library"):
        kernels.product_choices = {key: forced for key in table}
        products()
    path = str(tmp_path / "choices.json")
    kernels.save_product_choices(path)
    assert HipKernels.load_product_choices(path) == kernels.product_choices
    assert HipKernels("cuda:0", product_choices=HipKernels.load_product_choices(path)).product_choices == kernels.product_choices


MID_CASES = [  # rows, outs, k: every row-tile count, several blocks of rows, ragged k and outs, long and short k
    (17, 100, 72), (20, 304, 520), (33, 48, 2048), (50, 4096, 4096), (64, 320, 256), (100, 4096, 4096),
    (128, 520, 1032), (300, 1000, 2048), (512, 1536, 512), (48, 640, 12288), (5, 64, 32),
    (70, 264, 1032), (90, 4096, 512), (132, 520, 2048), (200, 304, 4096),      # five to seven tiles of rows a block
]


@pytest.mark.parametrize("rows,outs,k", MID_CASES)
def test_mid_size_product(hip_own, ref, rows, outs, k):
    """`akv_linear_mid` alone, with every cut it can be told to make (waves along a band, row tiles per wave, depth of
    the weight ring, blocks along k) and the cut it chooses itself, into bfloat16 and float32; twice each, since a
    launch that cuts k over blocks must leave its counters at zero for the next."""
    import ctypes
    from ampere_kv_engine_amd.kernels.hip import _ptr
    lib = hip_own.lib
    w = rand(outs, k, dtype=torch.bfloat16, seed=81, scale=0.05)
    x = rand(rows, k, dtype=torch.bfloat16, seed=82)
    packed = hip_own.prepare_linear(w.cuda())
    want = x.float() @ w.float().T
    partial = torch.empty(8 << 20, dtype=torch.float32, device="cuda")
    counters = torch.zeros(4096, dtype=torch.int32, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    xd = x.cuda()
    bias = rand(outs, seed=83, scale=0.5)
    bias_d = bias.cuda()
    plain_want = want
    for along, rt, depth, parts in ((0, 0, 0, 0), (2, 1, 4, 1), (3, 2, 2, 2), (4, 1, 4, 4), (4, 2, 2, 8), (3, 1, 0, 1), (2, 2, 0, 2)):
        for code, dtype in ((1, torch.bfloat16), (0, torch.float32)):
            for with_bias in (False, True):     # (twice: a launch that cuts k over blocks leaves its counters at zero)
                want = plain_want + bias if with_bias else plain_want
                got = torch.full((rows, outs), float("nan"), dtype=dtype, device="cuda")
                status = lib.akv_linear_mid(_ptr(xd), _ptr(packed.data), _ptr(got), code, _ptr(partial), ctypes.c_long(partial.numel()), _ptr(counters), ctypes.c_long(counters.numel()), rows,
                                            outs, k, packed.n_tiles, packed.k_tiles, 0, along, rt, depth, parts, _ptr(bias_d) if with_bias else None, stream)
                assert status == 0, (along, rt, depth, parts, status)
                limits = tol(dtype) if dtype == torch.bfloat16 else dict(rtol=2e-5, atol=2e-5 * float(want.abs().max()))
                torch.testing.assert_close(got.cpu().float(), want if dtype == torch.float32 else want.bfloat16().float(), **limits,
                                           msg=lambda m: f"along {along} rt {rt} depth {depth} parts {parts} {dtype}: {m}")
            assert int(counters.abs().sum()) == 0
    # what is cut over blocks is added in the order of the parts, whoever comes last: two launches agree bit for bit
    first = torch.empty((rows, outs), dtype=torch.float32, device="cuda")
    again = torch.empty((rows, outs), dtype=torch.float32, device="cuda")
    for target in (first, again):
        assert lib.akv_linear_mid(_ptr(xd), _ptr(packed.data), _ptr(target), 0, _ptr(partial), ctypes.c_long(partial.numel()), _ptr(counters), ctypes.c_long(counters.numel()), rows, outs, k,
                                  packed.n_tiles, packed.k_tiles, 0, 4, 1, 4, 4, None, stream) == 0
    assert torch.equal(first, again)
    # a ring depth that the row tiles per wave do not allow is refused
    assert lib.akv_linear_mid(_ptr(xd), _ptr(packed.data), _ptr(first), 0, _ptr(partial), ctypes.c_long(partial.numel()), _ptr(counters),
                              ctypes.c_long(counters.numel()), rows, outs, k, packed.n_tiles, packed.k_tiles, 0, 2, 2, 4, 1, None, stream) == -2
    # a workspace that is too small for the cut is refused before anything is launched
    need, words = ctypes.c_long(0), ctypes.c_long(0)
    lib.akv_linear_mid_workspace(rows, packed.n_tiles, packed.k_tiles, 0, 4, 1, 4, 4, ctypes.byref(need), ctypes.byref(words))
    assert lib.akv_linear_mid(_ptr(xd), _ptr(packed.data), _ptr(first), 0, _ptr(partial), ctypes.c_long(16), _ptr(counters),
                              ctypes.c_long(counters.numel()), rows, outs, k, packed.n_tiles, packed.k_tiles, 0, 4, 1, 4, 4,
                              None, stream) == (-3 if need.value > 16 else 0)


@pytest.mark.parametrize("rows,inter,k", [(40, 208, 264), (64, 512, 2048), (130, 208, 520), (17, 16, 8), (256, 1024, 1024),
                                          (96, 512, 1032), (110, 208, 2048)])
def test_mid_size_gated_product(hip_own, ref, rows, inter, k):
    import ctypes
    from ampere_kv_engine_amd.kernels.hip import _ptr
    lib = hip_own.lib
    gate, up = (rand(inter, k, dtype=torch.bfloat16, seed=91 + i, scale=0.05) for i in range(2))
    x = rand(rows, k, dtype=torch.bfloat16, seed=93)
    weight = hip_own.prepare_gated_linear(gate.cuda(), up.cuda())
    want = torch.empty(rows, inter, dtype=torch.bfloat16)
    ref.gated_linear(x, ref.prepare_gated_linear(gate, up), want)
    partial = torch.empty(8 << 20, dtype=torch.float32, device="cuda")
    counters = torch.zeros(4096, dtype=torch.int32, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for along, parts in ((0, 0), (2, 1), (3, 2), (4, 4)):
        got = torch.full((rows, inter), float("nan"), dtype=torch.bfloat16, device="cuda")
        assert lib.akv_linear_mid(_ptr(x.cuda()), _ptr(weight.packed.data), _ptr(got), 1, _ptr(partial), ctypes.c_long(partial.numel()), _ptr(counters), ctypes.c_long(counters.numel()), rows,
                                  inter, k, weight.packed.n_tiles, weight.packed.k_tiles, 1, along, 2, 2, parts, None, stream) == 0
        torch.testing.assert_close(got.cpu().float(), want.float(), **tol(torch.bfloat16))
    assert int(counters.abs().sum()) == 0


@pytest.mark.parametrize("rows,hidden,k,inter", [(17, 96, 72, 64), (40, 304, 520, 208), (64, 1024, 2048, 512), (100, 4096, 4096, 1024),
                                                 (128, 520, 1032, 208), (132, 4096, 512, 512), (300, 1000, 2048, 256),
                                                 (512, 1536, 512, 128), (90, 5120, 256, 64), (200, 8192, 64, 32)])
def test_mid_size_products_keep_the_residual_sum_and_the_norm(hip_own, ref, rows, hidden, k, inter):
    """Steps of 17 to 512 rows: `add_to_stream` (stream += bfloat16(x W^T + b); leaves the new rows times the next
    norm's weight and, per band of its row tiles, the rows' sums of squares) and `linear_rowscaled` (the product of
    such rows, every result divided by its row's root mean square; plain with a bias, and gated) - each against its
    formula, the pair against the norm kernel followed by the ordinary products, and twice: the second call finds
    the counters of the first at zero and gives the same bits."""
    from ampere_kv_engine_amd.engine.batch import Arena
    eps = 1e-5
    w = rand(hidden, k, dtype=torch.bfloat16, seed=301, scale=0.05)
    x = rand(rows, k, dtype=torch.bfloat16, seed=302)
    bias = rand(hidden, seed=303, scale=0.5)
    before = rand(rows, hidden, seed=304, scale=2.0)
    gain = rand(hidden, seed=305).abs() + 0.5
    packed = hip_own.prepare_linear(w.cuda())
    arena = Arena("cuda:0")
    assert hip_own.adds_to_stream(rows, packed, torch.bfloat16, gain.cuda())
    assert not hip_own.adds_to_stream(rows, packed, torch.bfloat16, None)      # without the next norm's weight: no
    assert not hip_own.adds_to_stream(513, packed, torch.bfloat16, gain.cuda())
    stream = before.clone().cuda()
    left = hip_own.add_to_stream(x.cuda(), packed, stream, arena, bias=bias.cuda(), gain=gain.cuda())
    product = (x.float() @ w.float().T + bias).bfloat16().float()
    torch.testing.assert_close((stream.cpu() - before), product, rtol=1.6e-2, atol=2e-3)   # (a sum's low bits go when it is added to 2.0)
    now = stream.cpu()
    assert torch.equal(left.rows.cpu(), (now * gain).bfloat16())                # the rows it left, from the sum it left
    assert left.gain is not None and left.sums.shape[1] == (rows + 15) // 16 * 16
    totals = left.sums.sum(0).cpu()
    torch.testing.assert_close(totals[:rows], (now * now).sum(-1), rtol=1e-5, atol=1e-6)
    assert float(totals[rows:].abs().sum()) == 0.0
    again = before.clone().cuda()
    left_again = hip_own.add_to_stream(x.cuda(), packed, again, arena, bias=bias.cuda(), gain=gain.cuda())
    assert torch.equal(again, stream) and torch.equal(left_again.rows, left.rows) and torch.equal(left_again.sums, left.sums)

    # the products that read such rows
    scale = torch.rsqrt(totals[:rows, None] / hidden + eps)
    rows_left = left.rows.cpu().float()
    normed = torch.empty(rows, hidden, dtype=torch.bfloat16)
    ref.add_rmsnorm(now.clone(), None, gain, eps, normed)                      # what a norm kernel would hand on
    second = rand(inter, hidden, dtype=torch.bfloat16, seed=306, scale=0.05)
    second_bias = rand(inter, seed=307, scale=0.5)
    plain = hip_own.prepare_linear(second.cuda())
    most = hip_own.lib.akv_linear_mid_most_groups(rows)
    assert hip_own.scales_rows_in_product(rows, plain, torch.bfloat16, left) == (left.sums.shape[0] <= most)
    if left.sums.shape[0] > most:       # more partial sums a row than the reading product's fetching waves hold:
        return                          # the parts then norm the rows with the norm's own kernel
    for with_bias in (False, True):
        got = torch.full((rows, inter), float("nan"), dtype=torch.bfloat16, device="cuda")
        hip_own.linear_rowscaled(left.rows, left.sums, eps, plain, got, bias=second_bias.cuda() if with_bias else None)
        want = rows_left @ second.float().T * scale + (second_bias if with_bias else 0.0)
        torch.testing.assert_close(got.cpu().float(), want.bfloat16().float(), **tol(torch.bfloat16))
        # against the ordinary pair (rows normed, rounded, weighted, rounded; then the product): every operand is
        # rounded elsewhere, so single outputs differ by what bfloat16 operands allow - over all of them, little
        ordinary = (normed.float() @ second.float().T + (second_bias if with_bias else 0.0)).bfloat16().float()
        apart = got.cpu().float() - ordinary
        assert float(apart.pow(2).mean().sqrt()) <= 2.0 ** -7 * float(ordinary.pow(2).mean().sqrt())
        assert float(apart.abs().max()) <= 2.0 ** -4 * float(ordinary.pow(2).mean().sqrt())
    gate, up = (rand(inter, hidden, dtype=torch.bfloat16, seed=308 + i, scale=0.05) for i in range(2))
    gated = hip_own.prepare_gated_linear(gate.cuda(), up.cuda())
    assert hip_own.scales_rows_in_product(rows, gated, torch.bfloat16, left)
    got = torch.full((rows, inter), float("nan"), dtype=torch.bfloat16, device="cuda")
    hip_own.linear_rowscaled(left.rows, left.sums, eps, gated, got)
    g, u = rows_left @ gate.float().T * scale, rows_left @ up.float().T * scale
    torch.testing.assert_close(got.cpu().float(), (g * torch.sigmoid(g) * u).bfloat16().float(), **tol(torch.bfloat16))
    first = got.clone()
    hip_own.linear_rowscaled(left.rows, left.sums, eps, gated, got)
    assert torch.equal(first, got)
    assert int(hip_own._mid_counters.abs().sum()) == 0 if hip_own._mid_counters is not None else True


@pytest.mark.parametrize("rows", [5, 16, 40, 130])
@pytest.mark.parametrize("outs", [100, 90, 35])
def test_adding_products_at_widths_that_are_no_multiple_of_four(hip_own, rows, outs, monkeypatch):
    """The adding products' epilogues element by element (the engine never asks for such widths - a product that
    reads the rows needs a width that is a multiple of 8 - but the entry points take them): the residual sum, the
    rows left and the sums of squares, at up to 16 rows and beyond."""
    from ampere_kv_engine_amd.engine.batch import Arena
    monkeypatch.setattr(hip_own, "fold_norms", True)
    k = 264
    w = rand(outs, k, dtype=torch.bfloat16, seed=501, scale=0.05)
    x = rand(rows, k, dtype=torch.bfloat16, seed=502)
    bias = rand(outs, seed=503, scale=0.5)
    before = rand(rows, outs, seed=504, scale=2.0)
    gain = rand(outs, seed=505).abs() + 0.5
    stream = before.clone().cuda()
    left = hip_own.add_to_stream(x.cuda(), hip_own.prepare_linear(w.cuda()), stream, Arena("cuda:0"), bias=bias.cuda(), gain=gain.cuda())
    product = (x.float() @ w.float().T + bias).bfloat16().float()
    torch.testing.assert_close(stream.cpu() - before, product, rtol=1.6e-2, atol=2e-3)
    now = stream.cpu()
    assert torch.equal(left.rows.cpu(), (now * gain).bfloat16())
    totals = left.sums.sum(0).cpu()
    torch.testing.assert_close(totals[:rows], (now * now).sum(-1), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("rows,hidden,k,inter", [(1, 96, 72, 64), (3, 304, 520, 208), (8, 4096, 4096, 1024), (16, 4096, 512, 512),
                                                 (5, 1000, 2048, 256), (16, 5120, 256, 64), (8, 104, 64, 32), (2, 8192, 1024, 128)])
def test_decode_products_leave_rows_for_a_product_that_scales_its_sums(hip, ref, rows, hidden, k, inter, monkeypatch):
    """Steps of up to 16 rows: `linear_adds(..., rows_out=, gain=)` adds to the residual sum exactly as without the
    two (the same bits, sums of squares included) and leaves the new rows times the next norm's weight;
    `linear_rowscaled` multiplies such rows and scales every sum by its row's 1 / rms - plain with and without a bias,
    with one and two row tiles a wave, and gated - against its formula and against the product that norms its rows
    itself (`linear_scaled`)."""
    monkeypatch.setattr(hip, "fold_norms", True)
    eps = 1e-5
    w = rand(hidden, k, dtype=torch.bfloat16, seed=401, scale=0.05)
    x = rand(rows, k, dtype=torch.bfloat16, seed=402)
    bias = rand(hidden, seed=403, scale=0.5)
    before = rand(rows, hidden, seed=404, scale=2.0)
    gain = rand(hidden, seed=405).abs() + 0.5
    packed = hip.prepare_linear(w.cuda())
    tiles = (hidden + 15) // 16
    plain_stream, plain_sums = before.clone().cuda(), torch.full((tiles, 16), float("nan"), device="cuda")
    hip.linear_adds(x.cuda(), packed, plain_stream, plain_sums, bias=bias.cuda())
    stream, sums = before.clone().cuda(), torch.full((tiles, 16), float("nan"), device="cuda")
    left = torch.full((rows, hidden), float("nan"), dtype=torch.bfloat16, device="cuda")
    hip.linear_adds(x.cuda(), packed, stream, sums, bias=bias.cuda(), rows_out=left, gain=gain.cuda())
    assert torch.equal(stream, plain_stream) and torch.equal(sums, plain_sums)
    now = stream.cpu()
    assert torch.equal(left.cpu(), (now * gain).bfloat16())
    from ampere_kv_engine_amd.parts.base import StreamSums
    handed = StreamSums(sums, rows=left, gain=gain)
    totals = sums.sum(0).cpu()
    scale = torch.rsqrt(totals[:rows, None] / hidden + eps)
    rows_left = left.cpu().float()
    second = rand(inter, hidden, dtype=torch.bfloat16, seed=406, scale=0.05)
    second_bias = rand(inter, seed=407, scale=0.5)
    plain = hip.prepare_linear(second.cuda())
    assert hip.scales_rows_in_product(rows, plain, torch.bfloat16, handed)
    for with_bias in (False, True):
        b = second_bias.cuda() if with_bias else None
        norming = None
        if hip.norms_rows_in_product(rows, plain, torch.bfloat16):     # (its normed rows must fit a compute unit's LDS)
            norming = torch.empty((rows, inter), dtype=torch.bfloat16, device="cuda")
            hip.linear_scaled(stream, sums, gain.cuda(), eps, plain, norming, bias=b)
        want = rows_left @ second.float().T * scale + (second_bias if with_bias else 0.0)
        for row_tiles in (0, 1, 2):
            got = torch.full((rows, inter), float("nan"), dtype=torch.bfloat16, device="cuda")
            hip.linear_rowscaled(left, sums, eps, plain, got, bias=b, row_tiles=row_tiles)
            torch.testing.assert_close(got.cpu().float(), want.bfloat16().float(), **tol(torch.bfloat16))
            if norming is not None:
                apart = got.float() - norming.float()      # operands rounded elsewhere: little over all outputs
                assert float(apart.pow(2).mean().sqrt()) <= 2.0 ** -7 * float(norming.float().pow(2).mean().sqrt())
    gate, up = (rand(inter, hidden, dtype=torch.bfloat16, seed=408 + i, scale=0.05) for i in range(2))
    gated = hip.prepare_gated_linear(gate.cuda(), up.cuda())
    assert hip.scales_rows_in_product(rows, gated, torch.bfloat16, handed)
    got = torch.full((rows, inter), float("nan"), dtype=torch.bfloat16, device="cuda")
    hip.linear_rowscaled(left, sums, eps, gated, got)
    g, u = rows_left @ gate.float().T * scale, rows_left @ up.float().T * scale
    torch.testing.assert_close(got.cpu().float(), (g * torch.sigmoid(g) * u).bfloat16().float(), **tol(torch.bfloat16))
    again = torch.empty_like(got)
    hip.linear_rowscaled(left, sums, eps, gated, again)
    assert torch.equal(got, again)


def test_linear_keeps_other_weights_row_major(hip):
    assert isinstance(hip.prepare_linear(torch.zeros(4, 12, dtype=torch.bfloat16, device="cuda")), torch.Tensor)   # k % 8
    assert isinstance(hip.prepare_linear(torch.zeros(4, 16, device="cuda")), torch.Tensor)                         # float32


def test_linear_rows_do_not_depend_on_the_batch(hip):
    """Float32: a row's result is bit-identical whether it is computed alone or among others."""
    x, w = rand(67, 300, seed=13).cuda(), rand(150, 300, seed=14).cuda()
    whole = torch.empty(67, 150, device="cuda")
    hip.linear(x, w, whole)
    for row in (0, 1, 63, 64, 66):
        alone = torch.empty(1, 150, device="cuda")
        hip.linear(x[row:row + 1].contiguous(), w, alone)
        assert torch.equal(alone[0], whole[row])


@pytest.mark.parametrize("inter", [200, 204, 203, 4096])     # widths in steps of 8, of 4 and of 1
@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu(hip, ref, dtype, inter):
    gate_up = rand(37, 2 * inter, dtype=dtype, seed=15, scale=2.0)
    want = torch.empty(37, inter, dtype=dtype)
    ref.swiglu(gate_up, want)
    got = torch.full((37, inter), float("nan"), dtype=dtype, device="cuda")
    hip.swiglu(gate_up.cuda(), got)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dtype))


@pytest.mark.parametrize("dim,theta", [(16, 1e4), (32, 1e6), (128, 1e6), (80, 5e5)])
def test_rope_table_and_rope(hip, ref, dim, theta):
    exponent = torch.arange(0, dim, 2, dtype=torch.int64).float() / dim
    inv_freq = 1.0 / (theta ** exponent)
    want = torch.empty(9000, dim // 2, 2)
    ref.rope_table(inv_freq, want)
    got = torch.empty(9000, dim // 2, 2, device="cuda")
    hip.rope_table(inv_freq.cuda(), got)
    torch.testing.assert_close(got.cpu(), want, rtol=0, atol=2e-6)       # sin/cos of angles up to 9000 rad
    for dtype in DTYPES:
        x = rand(5, 3, dim, dtype=dtype, seed=16)
        positions = torch.tensor([0, 1, 17, 4095, 8999], dtype=torch.int32)
        x_ref, x_hip = x.clone(), x.clone().cuda()
        ref.rope(x_ref, positions, want)
        hip.rope(x_hip, positions.cuda(), got)
        torch.testing.assert_close(x_hip.cpu().float(), x_ref.float(), **tol(dtype))
        torch.testing.assert_close(x_hip.cpu()[0], x[0], rtol=0, atol=0)          # position 0 leaves x as it is


def _pages(num_pages, kv_heads, page_size, dim, dtype):
    """Key pages [pages, kv_heads, page_size, dim] and value pages [pages, kv_heads, dim, page_size], NaN-filled."""
    k = torch.full((num_pages, kv_heads, page_size, dim), float("nan"), dtype=dtype)
    return k, torch.full((num_pages, kv_heads, dim, page_size), float("nan"), dtype=dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("q_heads,kv_heads,dim,page_size", [(4, 2, 16, 16), (6, 1, 32, 8), (8, 8, 128, 4), (5, 5, 80, 32),
                                                             (2, 1, 256, 16)])
@pytest.mark.parametrize("normed,rotated,written", [(True, True, True), (False, True, True), (True, False, True),
                                                    (True, True, False)])
def test_qk_norm_rope_write(hip, ref, dtype, q_heads, kv_heads, dim, page_size, normed, rotated, written):
    tokens, num_pages = 7, 6
    qkv = rand(tokens, (q_heads + 2 * kv_heads) * dim, dtype=dtype, seed=17)
    qw, kw = (1 + rand(dim, seed=18, scale=0.1), 1 + rand(dim, seed=19, scale=0.1)) if normed else (None, None)
    exponent = torch.arange(0, dim, 2, dtype=torch.int64).float() / dim
    table = torch.empty(300, dim // 2, 2)
    ref.rope_table(1.0 / (1e4 ** exponent), table)
    positions = torch.tensor([0, 1, 2, 100, 101, 299, 7], dtype=torch.int32)
    # slots in reversed page order, crossing a page edge, leaving the others untouched
    slots = torch.tensor([5 * page_size + page_size - 1, 4 * page_size, 4 * page_size + 1, 2 * page_size + 3 % page_size,
                          1 * page_size, 0, 3 * page_size + page_size - 1], dtype=torch.int32)
    k_ref, v_ref = _pages(num_pages, kv_heads, page_size, dim, dtype)
    q_ref = torch.empty(tokens, q_heads * dim, dtype=dtype)
    ref.qk_norm_rope_write(qkv, qw, kw, 1e-6, table if rotated else None, positions, slots if written else None,
                           k_ref, v_ref, q_ref, q_heads, kv_heads, dim)
    k_hip, v_hip = (t.cuda() for t in _pages(num_pages, kv_heads, page_size, dim, dtype))
    q_hip = torch.empty(tokens, q_heads * dim, dtype=dtype, device="cuda")
    cu = lambda t: t.cuda() if t is not None else None
    hip.qk_norm_rope_write(qkv.cuda(), cu(qw), cu(kw), 1e-6, cu(table) if rotated else None, positions.cuda(),
                           slots.cuda() if written else None, k_hip, v_hip, q_hip, q_heads, kv_heads, dim)
    torch.testing.assert_close(q_hip.cpu().float(), q_ref.float(), **tol(dtype))
    torch.testing.assert_close(k_hip.cpu().float(), k_ref.float(), equal_nan=True, **tol(dtype))
    torch.testing.assert_close(v_hip.cpu().float(), v_ref.float(), equal_nan=True, rtol=0, atol=0)   # v: bitwise copy
    assert torch.isnan(k_hip.cpu().float()).sum() == torch.isnan(k_ref.float()).sum()   # nothing else was written


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("q_heads,kv_heads,dim,page_size", [(4, 2, 16, 16), (6, 1, 32, 8), (8, 8, 128, 4), (5, 5, 80, 32),
                                                             (2, 1, 256, 16), (32, 8, 128, 16)])
def test_qk_norm_rope_write_of_many_tokens(hip, ref, dtype, q_heads, kv_heads, dim, page_size):
    """From eight tokens on the values get blocks of their own that take eight rows at a time: eight slots that follow
    each other from a multiple of eight (one 16-byte store per dim), the same run shifted by three (it crosses into
    another page where pages are small), slots in falling order, a run cut by the end of the step."""
    starts = [4 * 64, 2 * 64 + 3, None, 5 * 64 + 8, 1 * 64]            # first slot of each group of eight rows
    slots = []
    for group, start in enumerate(starts):
        slots += [6 * 64 + 40 - 3 * i for i in range(8)] if start is None else [start + i for i in range(8)]
    slots = slots[:37]                                                   # the last group has five rows
    tokens, num_pages = len(slots), 8 * 64 // page_size
    qkv = rand(tokens, (q_heads + 2 * kv_heads) * dim, dtype=dtype, seed=51)
    qw, kw = 1 + rand(dim, seed=18, scale=0.1), 1 + rand(dim, seed=19, scale=0.1)
    exponent = torch.arange(0, dim, 2, dtype=torch.int64).float() / dim
    table = torch.empty(64, dim // 2, 2)
    ref.rope_table(1.0 / (1e4 ** exponent), table)
    positions = torch.arange(tokens, dtype=torch.int32) + 11
    slots = torch.tensor(slots, dtype=torch.int32)
    k_ref, v_ref = _pages(num_pages, kv_heads, page_size, dim, dtype)
    q_ref = torch.empty(tokens, q_heads * dim, dtype=dtype)
    ref.qk_norm_rope_write(qkv, qw, kw, 1e-6, table, positions, slots, k_ref, v_ref, q_ref, q_heads, kv_heads, dim)
    k_hip, v_hip = (t.cuda() for t in _pages(num_pages, kv_heads, page_size, dim, dtype))
    q_hip = torch.empty(tokens, q_heads * dim, dtype=dtype, device="cuda")
    hip.qk_norm_rope_write(qkv.cuda(), qw.cuda(), kw.cuda(), 1e-6, table.cuda(), positions.cuda(), slots.cuda(), k_hip,
                           v_hip, q_hip, q_heads, kv_heads, dim)
    torch.testing.assert_close(q_hip.cpu().float(), q_ref.float(), **tol(dtype))
    torch.testing.assert_close(k_hip.cpu().float(), k_ref.float(), equal_nan=True, **tol(dtype))
    torch.testing.assert_close(v_hip.cpu().float(), v_ref.float(), equal_nan=True, rtol=0, atol=0)   # v: bitwise copy
    assert torch.isnan(v_hip.cpu().float()).sum() == torch.isnan(v_ref.float()).sum()   # nothing else was written


@pytest.mark.parametrize("dtype", DTYPES)
def test_kv_write(hip, ref, dtype):
    tokens, kv_heads, dim, page_size = 5, 3, 48, 8
    k = rand(tokens, kv_heads, dim, dtype=dtype, seed=20)
    wide = rand(tokens, 5 * kv_heads * dim, dtype=dtype, seed=21)
    v = wide[:, kv_heads * dim:2 * kv_heads * dim].unflatten(1, (kv_heads, dim))
    slots = torch.tensor([15, 16, 0, 31, 9], dtype=torch.int32)
    k_ref, v_ref = _pages(4, kv_heads, page_size, dim, dtype)
    ref.kv_write(k, v, slots, k_ref, v_ref)
    k_hip, v_hip = (t.cuda() for t in _pages(4, kv_heads, page_size, dim, dtype))
    hip.kv_write(k.cuda(), wide.cuda()[:, kv_heads * dim:2 * kv_heads * dim].unflatten(1, (kv_heads, dim)), slots.cuda(),
                 k_hip, v_hip)
    torch.testing.assert_close(k_hip.cpu().float(), k_ref.float(), equal_nan=True, rtol=0, atol=0)
    torch.testing.assert_close(v_hip.cpu().float(), v_ref.float(), equal_nan=True, rtol=0, atol=0)


def _attention_case(dtype, q_heads, kv_heads, dim, page_size, portions, window, seed, spike=None):
    """`portions` = [(history, new tokens)] per request.  Pages are handed out in a scrambled order; pages a
    window has passed and table padding hold -1; unwritten slots hold NaN."""
    g = torch.Generator().manual_seed(seed)
    lengths = [h + n for h, n in portions]
    pages_of = [math.ceil(l / page_size) for l in lengths]
    num_pages = sum(pages_of) + 3
    order = torch.randperm(num_pages, generator=g).tolist()
    k_pages, v_pages = _pages(num_pages, kv_heads, page_size, dim, dtype)
    width = max(pages_of) + 1
    table = torch.full((len(portions), width), -1, dtype=torch.int32)
    keys, values = [], []
    cursor = 0
    for r, length in enumerate(lengths):
        k = torch.randn(length, kv_heads, dim, generator=g).to(dtype)
        v = torch.randn(length, kv_heads, dim, generator=g).to(dtype)
        if spike is not None and r == spike[0]:
            k[spike[1]] *= 6.0       # one far key stands out of hundreds
        keys.append(k)
        values.append(v)
        history = portions[r][0]
        lowest = 0 if window is None else max(0, history - window + 1)
        for p in range(pages_of[r]):
            page = order[cursor]
            cursor += 1
            if (p + 1) * page_size <= lowest:
                continue               # wholly passed by the window: given back, entry stays -1
            table[r, p] = page
            lo, hi = p * page_size, min((p + 1) * page_size, length)
            k_pages[page, :, :hi - lo] = k[lo:hi].transpose(0, 1)
            v_pages[page, :, :, :hi - lo] = v[lo:hi].permute(1, 2, 0)
    tokens = sum(n for _, n in portions)
    q = torch.randn(tokens, q_heads * dim, generator=g).to(dtype)
    if spike is not None:
        r, at = spike
        first = sum(n for _, n in portions[:r])
        q[first:first + portions[r][1]] = (keys[r][at].float().repeat(q_heads // kv_heads, 1).reshape(-1) * 2.0).to(dtype)
    q_start = [0]
    for _, n in portions:
        q_start.append(q_start[-1] + n)
    positions = torch.cat([torch.arange(h, h + n) for h, n in portions]).int()
    seq_of_token = torch.cat([torch.full((n,), r) for r, (_, n) in enumerate(portions)]).int()
    ctx = SimpleNamespace(num_seqs=len(portions), num_tokens=tokens, host_q_start=q_start, host_seq_lens=lengths,
                          positions=positions, seq_of_token=seq_of_token, max_seq_len=max(lengths),
                          num_decode_seqs=0, max_new_tokens=max(n for _, n in portions))
    meta = SimpleNamespace(block_table=table, width=width, window=window)
    return q, k_pages, v_pages, ctx, meta, keys, values


def _to_cuda(ctx, meta):
    c = SimpleNamespace(**vars(ctx))
    c.positions, c.seq_of_token = ctx.positions.cuda(), ctx.seq_of_token.cuda()
    c.q_start = torch.tensor(ctx.host_q_start, dtype=torch.int32, device="cuda")
    c.seq_lens = torch.tensor(ctx.host_seq_lens, dtype=torch.int32, device="cuda")
    m = SimpleNamespace(**vars(meta))
    m.block_table = meta.block_table.cuda()
    return c, m


ATTENTION_SIZES = [(4, 2, 16, 16), (6, 1, 32, 8), (8, 2, 128, 16), (5, 5, 80, 4), (3, 1, 256, 32)]
PORTIONS = [[(0, 1)], [(0, 33)], [(64, 1), (17, 1), (0, 1)], [(5, 7), (63, 2), (130, 1), (0, 70)]]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("q_heads,kv_heads,dim,page_size", ATTENTION_SIZES)
@pytest.mark.parametrize("portions", PORTIONS)
@pytest.mark.parametrize("window", [None, 24])
def test_attention(hip, ref, dtype, q_heads, kv_heads, dim, page_size, portions, window):
    q, k_pages, v_pages, ctx, meta, _, _ = _attention_case(dtype, q_heads, kv_heads, dim, page_size, portions, window, 22)
    want = torch.empty_like(q)
    ref.attention(q, k_pages, v_pages, ctx, meta, q_heads, kv_heads, dim, dim ** -0.5, window, want)
    cctx, cmeta = _to_cuda(ctx, meta)
    got = torch.empty_like(q, device="cuda")
    hip.attention(q.cuda(), k_pages.cuda(), v_pages.cuda(), cctx, cmeta, q_heads, kv_heads, dim, dim ** -0.5, window, got)
    assert not torch.isnan(got).any()
    torch.testing.assert_close(got.cpu().float(), want.float(), **attention_tol(dtype))


@pytest.mark.parametrize("shared", ["narrow", "wide", False, "cut"])
@pytest.mark.parametrize("q_heads,kv_heads,dim,page_size", [(8, 2, 128, 16), (6, 1, 32, 8), (8, 4, 64, 64), (3, 1, 256, 32),
                                                            (5, 5, 80, 16), (40, 2, 64, 8), (4, 2, 16, 128)])
@pytest.mark.parametrize("portions", [[(0, 700)], [(100, 300), (0, 45), (511, 2)]])
@pytest.mark.parametrize("window", [None, 100])
def test_attention_prompt_portions(hip, ref, shared, q_heads, kv_heads, dim, page_size, portions, window):
    """Long portions on the bfloat16 prompt kernels: blocks of four waves that share keys and values through LDS, with
    16 and with 32 columns per wave (several blocks per request, steps inside one page and across four, groups of
    more heads than a tile), one wave per tile, and one wave per tile and segment of the keys (what short portions
    after long histories get)."""
    q, k_pages, v_pages, ctx, meta, _, _ = _attention_case(torch.bfloat16, q_heads, kv_heads, dim, page_size, portions,
                                                           window, 28)
    want = torch.empty_like(q)
    ref.attention(q, k_pages, v_pages, ctx, meta, q_heads, kv_heads, dim, dim ** -0.5, window, want)
    cctx, cmeta = _to_cuda(ctx, meta)
    got = torch.full_like(q, float("nan"), device="cuda")
    hip.share_prompt_tiles, hip.wide_prompt_tiles, hip.split_prompt_keys = bool(shared), shared == "wide", shared == "cut"
    hip.decode_min_segment = 32 if shared == "cut" else hip.decode_min_segment    # several segments at these lengths
    try:
        hip.attention(q.cuda(), k_pages.cuda(), v_pages.cuda(), cctx, cmeta, q_heads, kv_heads, dim, dim ** -0.5, window, got)
    finally:
        hip.share_prompt_tiles, hip.wide_prompt_tiles, hip.split_prompt_keys, hip.decode_min_segment = True, None, None, 128
    torch.testing.assert_close(got.cpu().float(), want.float(), **attention_tol(torch.bfloat16))


@pytest.mark.parametrize("q_heads,kv_heads,dim,page_size", ATTENTION_SIZES + [(32, 8, 128, 16), (40, 2, 64, 8)])
@pytest.mark.parametrize("histories", [[0], [64, 17, 0], [1500, 2, 700, 255], [4000] * 9])
@pytest.mark.parametrize("window", [None, 100])
def test_attention_decode_batch(hip, ref, q_heads, kv_heads, dim, page_size, histories, window):
    """Single tokens of several requests (the split-key path of the bfloat16 kernel), histories from nothing to
    thousands of keys, more heads per group than one tile holds."""
    portions = [(h, 1) for h in histories]
    q, k_pages, v_pages, ctx, meta, _, _ = _attention_case(torch.bfloat16, q_heads, kv_heads, dim, page_size, portions,
                                                           window, 25)
    ctx.num_decode_seqs = len(portions)
    want = torch.empty_like(q)
    ref.attention(q, k_pages, v_pages, ctx, meta, q_heads, kv_heads, dim, dim ** -0.5, window, want)
    cctx, cmeta = _to_cuda(ctx, meta)
    got = torch.empty_like(q, device="cuda")
    hip.attention(q.cuda(), k_pages.cuda(), v_pages.cuda(), cctx, cmeta, q_heads, kv_heads, dim, dim ** -0.5, window, got)
    assert not torch.isnan(got).any()
    torch.testing.assert_close(got.cpu().float(), want.float(), **attention_tol(torch.bfloat16))


@pytest.mark.parametrize("lengths,window", [([9000, 130, 129, 4000], None), ([300] * 64, None), ([70000, 33, 512], None),
                                            ([5000, 200, 1000], 300), ([1], None)])
def test_decode_plan(hip, lengths, window):
    """The cut of single tokens' keys into items, as the one-wave kernel writes it, against the rule in plain
    arithmetic: one segment size for all requests from the sum of their spans, items numbered request by request."""
    items_wanted, smallest, first_request = 256, 128, 2
    seq_lens = torch.tensor([7, 7] + lengths, dtype=torch.int32, device="cuda")        # two requests before the launch's
    ctx = SimpleNamespace(seq_lens=seq_lens, num_seqs=len(lengths) + 2, host_seq_lens=[7, 7] + lengths)
    hip.decode_wave_target, kept = items_wanted * 4, hip.decode_wave_target
    try:
        plan, grid = hip._decode_plan(ctx, first_request, len(lengths), window, 4)
    finally:
        hip.decode_wave_target = kept
    plan = plan.cpu().tolist()
    spans, firsts = [], []
    for length in lengths:
        pos = length - 1
        first = (max(0, pos - window + 1) if window else 0) // 32 * 32
        firsts.append(first)
        spans.append(pos - first + 1)
    size = max(smallest, (-(-sum(spans) // items_wanted) + 31) // 32 * 32)
    counts = [-(-span // size) for span in spans]
    assert plan[0] == sum(counts) <= grid and plan[1] == size
    item = 0
    for r, (length, first, count) in enumerate(zip(lengths, firsts, counts)):
        assert plan[4 + 2 * r:6 + 2 * r] == [item, count]
        for z in range(count):
            lo = first + z * size
            assert plan[132 + 4 * item:136 + 4 * item] == [r, lo, length - 1, min(length - 1, lo + size - 1)]
            item += 1


def test_attention_of_many_single_tokens_of_very_different_lengths(hip, ref):
    """70 requests in one step (two launches of at most 64), one of them a hundred times longer than most: every
    request's keys are cut into segments of the same size."""
    histories = [6000] + [40 + 13 * i for i in range(69)]
    portions = [(h, 1) for h in histories]
    q, k_pages, v_pages, ctx, meta, _, _ = _attention_case(torch.bfloat16, 8, 2, 128, 16, portions, None, 36)
    ctx.num_decode_seqs = len(portions)
    want = torch.empty_like(q)
    ref.attention(q, k_pages, v_pages, ctx, meta, 8, 2, 128, 128 ** -0.5, None, want)
    cctx, cmeta = _to_cuda(ctx, meta)
    got = torch.full_like(q, float("nan"), device="cuda")
    hip.attention(q.cuda(), k_pages.cuda(), v_pages.cuda(), cctx, cmeta, 8, 2, 128, 128 ** -0.5, None, got)
    torch.testing.assert_close(got.cpu().float(), want.float(), **attention_tol(torch.bfloat16))
    assert len(cctx.decode_plans) == 2


def test_short_portion_after_a_long_history_has_its_keys_cut(hip, ref):
    """16 tokens after 2,500: blocks of four tiles would be 16 on the whole device, so the keys are cut over waves
    (the same request beside a single token of another; the rule is asked directly too)."""
    portions = [(700, 1), (2500, 16)]
    q, k_pages, v_pages, ctx, meta, _, _ = _attention_case(torch.bfloat16, 8, 2, 128, 16, portions, None, 33)
    ctx.num_decode_seqs = 1
    assert hip._few_portion_blocks(ctx, 1, 8, 2)
    long_portion = SimpleNamespace(host_q_start=[0, 1, 2049], num_seqs=2, max_seq_len=4096, host_seq_lens=[700, 4096])
    assert not hip._few_portion_blocks(long_portion, 1, 8, 2)
    # the history that counts is the portion's own request's, not that of a single token beside it
    beside_long = SimpleNamespace(host_q_start=[0, 1, 17], num_seqs=2, max_seq_len=9000, host_seq_lens=[9000, 500])
    assert not hip._few_portion_blocks(beside_long, 1, 8, 2)
    want = torch.empty_like(q)
    ref.attention(q, k_pages, v_pages, ctx, meta, 8, 2, 128, 128 ** -0.5, None, want)
    cctx, cmeta = _to_cuda(ctx, meta)
    got = torch.full_like(q, float("nan"), device="cuda")
    hip.attention(q.cuda(), k_pages.cuda(), v_pages.cuda(), cctx, cmeta, 8, 2, 128, 128 ** -0.5, None, got)
    torch.testing.assert_close(got.cpu().float(), want.float(), **attention_tol(torch.bfloat16))


def test_attention_decodes_beside_portions(hip, ref):
    """A mixed step: three single tokens first, then two portions; both launches write their own rows only."""
    portions = [(300, 1), (15, 1), (0, 1), (40, 37), (0, 130)]
    q, k_pages, v_pages, ctx, meta, _, _ = _attention_case(torch.bfloat16, 8, 2, 128, 16, portions, None, 26)
    ctx.num_decode_seqs = 3
    want = torch.empty_like(q)
    ref.attention(q, k_pages, v_pages, ctx, meta, 8, 2, 128, 128 ** -0.5, None, want)
    cctx, cmeta = _to_cuda(ctx, meta)
    got = torch.full_like(q, float("nan"), device="cuda")
    hip.attention(q.cuda(), k_pages.cuda(), v_pages.cuda(), cctx, cmeta, 8, 2, 128, 128 ** -0.5, None, got)
    torch.testing.assert_close(got.cpu().float(), want.float(), **attention_tol(torch.bfloat16))


def _raw_projection_case(q_heads, kv_heads, dim, page_size, portions, window, seed, decodes):
    """An attention case whose new tokens are not in the cache yet: their slots hold NaN, their stacked raw
    projections come beside, with the slot of every token as the block tables name it."""
    _, k_pages, v_pages, ctx, meta, _, _ = _attention_case(torch.bfloat16, q_heads, kv_heads, dim, page_size, portions,
                                                           window, seed)
    ctx.num_decode_seqs = decodes
    slots = []
    for r, (history, new) in enumerate(portions):
        for pos in range(history, history + new):
            page = int(meta.block_table[r, pos // page_size])
            slots.append(page * page_size + pos % page_size)
            k_pages[page, :, pos % page_size] = float("nan")
            v_pages[page, :, :, pos % page_size] = float("nan")
    qkv = rand(ctx.num_tokens, (q_heads + 2 * kv_heads) * dim, dtype=torch.bfloat16, seed=seed + 1)
    exponent = torch.arange(0, dim, 2, dtype=torch.int64).float() / dim
    table = torch.empty(ctx.max_seq_len + 1, dim // 2, 2)
    TorchKernels().rope_table(1.0 / (1e4 ** exponent), table)
    return qkv, table, torch.tensor(slots, dtype=torch.int32), k_pages, v_pages, ctx, meta


def _check_encode_and_attend(hip, ref, q_heads, kv_heads, dim, page_size, portions, window, decodes, normed=True,
                             rotated=True, seed=31):
    qkv, table, slots, k_pages, v_pages, ctx, meta = _raw_projection_case(q_heads, kv_heads, dim, page_size, portions,
                                                                          window, seed, decodes)
    qw, kw = (1 + rand(dim, seed=18, scale=0.1), 1 + rand(dim, seed=19, scale=0.1)) if normed else (None, None)
    sizes = (q_heads, kv_heads, dim, dim ** -0.5, window)
    k_ref, v_ref = k_pages.clone(), v_pages.clone()
    want = torch.empty(ctx.num_tokens, q_heads * dim, dtype=torch.bfloat16)
    ref.encode_and_attend(qkv, qw, kw, 1e-6, table if rotated else None, ctx.positions, slots, k_ref, v_ref,
                          torch.empty_like(want), ctx, meta, *sizes, want)
    cctx, cmeta = _to_cuda(ctx, meta)
    cu = lambda t: t.cuda() if t is not None else None
    k_hip, v_hip = k_pages.cuda(), v_pages.cuda()
    got = torch.full_like(want, float("nan"), device="cuda")
    hip.encode_and_attend(qkv.cuda(), cu(qw), cu(kw), 1e-6, cu(table) if rotated else None, cctx.positions, slots.cuda(),
                          k_hip, v_hip, torch.empty_like(got), cctx, cmeta, *sizes, got)
    assert not torch.isnan(got).any()
    torch.testing.assert_close(got.cpu().float(), want.float(), **attention_tol(torch.bfloat16))
    torch.testing.assert_close(k_hip.cpu().float(), k_ref.float(), equal_nan=True, **tol(torch.bfloat16))
    torch.testing.assert_close(v_hip.cpu().float(), v_ref.float(), equal_nan=True, rtol=0, atol=0)
    assert torch.isnan(k_hip.cpu().float()).sum() == torch.isnan(k_ref.float()).sum()   # nothing else was written


@pytest.mark.parametrize("q_heads,kv_heads,dim,page_size", [(8, 2, 128, 16), (4, 4, 64, 4), (40, 2, 64, 8), (3, 1, 256, 32),
                                                            (6, 2, 192, 16), (6, 1, 32, 8), (5, 5, 80, 16)])
@pytest.mark.parametrize("histories", [[0], [31, 32, 63, 64, 15, 16, 1], [1500, 2, 700, 255, 1023], [4000] * 9])
@pytest.mark.parametrize("window", [None, 100])
def test_encode_and_attend_single_tokens(hip, ref, q_heads, kv_heads, dim, page_size, histories, window):
    """Single tokens whose projections are raw: head sizes that are multiples of 64 go through the attention kernel
    that norms, rotates and writes them itself (positions at the first and last key of a step, of a page and of a
    segment; more heads per group than a tile holds), the others through the two kernels."""
    _check_encode_and_attend(hip, ref, q_heads, kv_heads, dim, page_size, [(h, 1) for h in histories], window,
                             len(histories))


@pytest.mark.parametrize("normed,rotated", [(False, True), (True, False), (False, False)])
def test_encode_and_attend_without_norm_or_rotation(hip, ref, normed, rotated):
    _check_encode_and_attend(hip, ref, 8, 2, 128, 16, [(h, 1) for h in (300, 0, 77)], None, 3, normed, rotated)


@pytest.mark.parametrize("dim", [128, 80])
def test_encode_and_attend_mixed_step(hip, ref, dim):
    """Three single tokens first, then two portions: the portions' rows alone go through the encoding kernel."""
    _check_encode_and_attend(hip, ref, 8, 2, dim, 16, [(300, 1), (15, 1), (0, 1), (40, 37), (0, 130)], None, 3)


def test_encode_and_attend_is_the_two_kernels(hip, ref):
    """The attention kernel's own encoding gives what the encoding kernel followed by the attention gives, to the
    rounding of the head's sum of squares (another order of the same sum)."""
    portions = [(h, 1) for h in (2000, 33, 0, 640)]
    qkv, table, slots, k_pages, v_pages, ctx, meta = _raw_projection_case(8, 2, 128, 16, portions, None, 35, 4)
    qw, kw = 1 + rand(128, seed=18, scale=0.1), 1 + rand(128, seed=19, scale=0.1)
    cctx, cmeta = _to_cuda(ctx, meta)
    outs = []
    for fresh in (True, False):
        hip.fresh_decode_tokens = fresh
        try:
            k_hip, v_hip = k_pages.cuda(), v_pages.cuda()
            got = torch.empty(4, 8 * 128, dtype=torch.bfloat16, device="cuda")
            hip.encode_and_attend(qkv.cuda(), qw.cuda(), kw.cuda(), 1e-6, table.cuda(), cctx.positions, slots.cuda(),
                                  k_hip, v_hip, torch.empty_like(got), cctx, cmeta, 8, 2, 128, 128 ** -0.5, None, got)
            outs.append((got.float().cpu(), k_hip.float().cpu(), v_hip.float().cpu()))
        finally:
            hip.fresh_decode_tokens = True
    torch.testing.assert_close(outs[0][0], outs[1][0], rtol=0.01, atol=0.002)
    torch.testing.assert_close(outs[0][1], outs[1][1], equal_nan=True, rtol=1e-2, atol=1e-3)
    assert (outs[0][1].nan_to_num() != outs[1][1].nan_to_num()).float().mean() < 0.01   # nearly every key bit for bit
    torch.testing.assert_close(outs[0][2], outs[1][2], equal_nan=True, rtol=0, atol=0)


def test_attention_over_a_pool_of_more_than_4_gb(hip, ref):
    """The request's pages lie at the end of a pool whose key tensor alone has 4.6 GB: page offsets need 64 bits.
    One single token (split-key kernel) and one prompt portion (shared-tile kernel)."""
    q_heads, kv_heads, dim, page_size = 8, 8, 128, 16
    portions = [(300, 1), (0, 150)]
    q, k_pages, v_pages, ctx, meta, _, _ = _attention_case(torch.bfloat16, q_heads, kv_heads, dim, page_size, portions, None, 29)
    ctx.num_decode_seqs = 1
    want = torch.empty_like(q)
    ref.attention(q, k_pages, v_pages, ctx, meta, q_heads, kv_heads, dim, dim ** -0.5, None, want)
    pool = 140_000                                     # x 32 KB per page and tensor
    shift = pool - k_pages.shape[0]
    k_big = torch.empty((pool, kv_heads, page_size, dim), dtype=torch.bfloat16, device="cuda")
    v_big = torch.empty((pool, kv_heads, dim, page_size), dtype=torch.bfloat16, device="cuda")
    assert k_big.numel() * 2 > 2 ** 32
    k_big[shift:] = k_pages.cuda()
    v_big[shift:] = v_pages.cuda()
    cctx, cmeta = _to_cuda(ctx, meta)
    cmeta.block_table = torch.where(cmeta.block_table >= 0, cmeta.block_table + shift, cmeta.block_table)
    got = torch.full_like(q, float("nan"), device="cuda")
    hip.attention(q.cuda(), k_big, v_big, cctx, cmeta, q_heads, kv_heads, dim, dim ** -0.5, None, got)
    torch.testing.assert_close(got.cpu().float(), want.float(), **attention_tol(torch.bfloat16))


def test_attention_poisons_a_foreign_page(hip):
    """A table entry inside a request's length that is no page of the pool gives NaN, not a read outside the pool."""
    portions = [(40, 1), (40, 5)]
    q, k_pages, v_pages, ctx, meta, _, _ = _attention_case(torch.bfloat16, 4, 2, 64, 16, portions, None, 27)
    ctx.num_decode_seqs = 1
    meta.block_table[0, 1] = -1
    meta.block_table[1, 0] = 10 ** 6
    cctx, cmeta = _to_cuda(ctx, meta)
    got = torch.zeros_like(q, device="cuda")
    hip.attention(q.cuda(), k_pages.cuda(), v_pages.cuda(), cctx, cmeta, 4, 2, 64, 64 ** -0.5, None, got)
    assert torch.isnan(got).all()


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_finds_a_far_key(hip, ref, dtype):
    """One key among a thousand matches the query: the output must be (nearly) that key's value."""
    portions = [(1000, 1), (900, 3)]
    for spike in ((0, 3), (1, 517)):
        q, k_pages, v_pages, ctx, meta, keys, values = _attention_case(dtype, 4, 2, 64, 16, portions, None, 23, spike)
        ctx.num_decode_seqs = 1            # the first request brings one token
        cctx, cmeta = _to_cuda(ctx, meta)
        got = torch.empty_like(q, device="cuda")
        hip.attention(q.cuda(), k_pages.cuda(), v_pages.cuda(), cctx, cmeta, 4, 2, 64, 64 ** -0.5, None, got)
        want = torch.empty_like(q)
        ref.attention(q, k_pages, v_pages, ctx, meta, 4, 2, 64, 64 ** -0.5, None, want)
        torch.testing.assert_close(got.cpu().float(), want.float(), **attention_tol(dtype))
        r, at = spike
        first = ctx.host_q_start[r]
        picked = got.cpu().float()[first].reshape(4, 64)
        torch.testing.assert_close(picked[0], values[r][at, 0].float(), rtol=0.05, atol=0.05)
        torch.testing.assert_close(picked[3], values[r][at, 1].float(), rtol=0.05, atol=0.05)


@pytest.mark.parametrize("portions,spike", [
    ([(120_000, 1), (300, 1), (70_001, 1)], (0, 5)),        # single tokens: 128 segments of a thousand keys; a far, early key
    ([(120_000, 1), (300, 1), (70_001, 1)], (2, 69_999)),   # ... and one in another request's last segment but one
    ([(60_000, 48)], (0, 59_000)),                          # a short portion after a long history: its keys are cut
    ([(0, 3_000)], (0, 7)),                                 # a long prompt whole: blocks of four waves, ninety calm steps
    ([(2_500, 700), (0, 40)], (0, 2_499)),                  # a long portion after a history, the key at the history's end
])
def test_attention_at_long_contexts_finds_a_far_key(hip, ref, portions, spike):
    """Qwen3-8B's head shape (four query heads to a key head of 128) at lengths far beyond the other tests', where a
    launch's cut of the keys, the calm steps of a long prompt and 32-bit offsets into a request's table are not what
    they are at a few hundred tokens.  The queries of the spiked request match one far key: their output is that
    key's value, and everything equals the torch double within the attention's limits."""
    q_heads, kv_heads, dim, page_size = 4, 1, 128, 16
    q, k_pages, v_pages, ctx, meta, keys, values = _attention_case(torch.bfloat16, q_heads, kv_heads, dim, page_size,
                                                                   portions, None, 31, spike)
    ctx.num_decode_seqs = sum(1 for _, n in portions if n == 1) if all(n == 1 for _, n in portions) else 0
    want = torch.empty_like(q)
    ref.attention(q, k_pages, v_pages, ctx, meta, q_heads, kv_heads, dim, dim ** -0.5, None, want)
    cctx, cmeta = _to_cuda(ctx, meta)
    got = torch.full_like(q, float("nan"), device="cuda")
    hip.attention(q.cuda(), k_pages.cuda(), v_pages.cuda(), cctx, cmeta, q_heads, kv_heads, dim, dim ** -0.5, None, got)
    torch.testing.assert_close(got.cpu().float(), want.float(), **attention_tol(torch.bfloat16))
    r, at = spike
    rows = range(ctx.host_q_start[r], ctx.host_q_start[r + 1])
    seen = [row for row in rows if int(ctx.positions[row]) >= at]           # (earlier tokens of a prompt cannot see it)
    assert seen
    for row in (seen[0], seen[-1]):
        torch.testing.assert_close(got.cpu().float()[row].reshape(q_heads, dim)[2], values[r][at, 0].float(), rtol=0.05, atol=0.05)


@pytest.mark.parametrize("vocab", [1531, 1532, 40004])     # single loads; 16-byte loads; more than one round of them
def test_sample(hip, vocab):
    import numpy as np
    logits = rand(6, vocab, seed=24, scale=2.0)
    logits[1, 100] = logits[1, 900] = 50.0                                  # a tie: the lowest id wins
    logits[5] = logits[2]
    temperature = torch.tensor([0.0, 0.0, 0.7, 0.7, 1.3, 0.7])
    seeds = torch.tensor([1, 2, 3, 3, (5 << 33) + 9, 3], dtype=torch.int64)
    draws = torch.tensor([0, 0, 0, 1, 7, 0], dtype=torch.int32)
    out = torch.empty(6, dtype=torch.int32, device="cuda")
    hip.sample(logits.cuda(), temperature.cuda(), seeds.cuda(), draws.cuda(), out)
    out = out.cpu().tolist()
    assert out[0] == int(logits[0].argmax()) and out[1] == 100
    assert out[2] == out[5]                                                   # same seed and draw: same token
    for row in (2, 3, 4):
        bits = philox_first(np.arange(vocab), int(draws[row]), int(seeds[row]) & 0xFFFFFFFF, int(seeds[row]) >> 32)
        u = ((bits >> np.uint64(8)).astype(np.float64) + 0.5) * 2.0 ** -24
        scores = logits[row].double().numpy() / float(temperature[row]) - np.log(-np.log(u))
        assert scores[out[row]] >= scores.max() - 1e-4
    greedy = torch.empty(6, dtype=torch.int32, device="cuda")
    hip.argmax(logits.cuda(), greedy)
    assert greedy.cpu().tolist() == [int(r.argmax()) if i != 1 else 100 for i, r in enumerate(logits)]


@pytest.mark.parametrize("rows,vocab", [(1, 151936), (3, 40004), (8, 151936), (64, 32768), (5, 8197), (300, 4096)])
def test_a_row_cut_over_several_blocks_chooses_what_one_block_chooses(hip, rows, vocab, monkeypatch):
    """Few rows of many logits are cut over several blocks a row, whose bests the last block of the row compares:
    greedy and with temperatures, ties within and across parts, a row with a NaN, a row of -inf - the tokens are
    those of the one-block kernel, twice in a row (the arrival counters are left at zero), handed in and from slots."""
    import struct
    generator = torch.Generator().manual_seed(rows * 7 + vocab)
    logits = torch.randn(rows, vocab, generator=generator) * 2
    logits[0, vocab - 1] = logits[0, 17] = 60.0                  # a tie across the row's ends: the lowest id
    if rows > 2:
        logits[1, vocab // 3] = float("nan")
        logits[2] = float("-inf")
    temperature = torch.tensor([0.0 if r % 2 == 0 else 0.5 + 0.1 * (r % 7) for r in range(rows)])
    seeds = torch.arange(rows, dtype=torch.int64) * 977 + (3 << 34)
    draws = torch.arange(rows, dtype=torch.int32) % 5
    on = [t.cuda() for t in (logits, temperature, seeds, draws)]
    monkeypatch.setattr(hip, "sample_in_parts", False)
    want = torch.empty(rows, dtype=torch.int32, device="cuda")
    hip.sample(*on, want)
    monkeypatch.setattr(hip, "sample_in_parts", True)
    assert (hip._sample_parts(rows, vocab) > 1) == (rows <= 128 and vocab >= 4096)
    for _ in range(200 if rows == 8 else 2):      # (back to back: whichever block of a row is last, the same token)
        got = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
        hip.sample(*on, got)
        assert torch.equal(got, want)
    assert want[0] == 17 and (rows <= 2 or (want[1] == -1 and want[2] == -1))
    if hip._sample_workspace is not None:
        assert int(hip._sample_workspace[2].abs().sum()) == 0
    # from slots: request r in slot rows - 1 - r, one token row each
    words = torch.zeros(rows, 8, dtype=torch.int32)
    for r in range(rows):
        seed = int(seeds[r])
        words[rows - 1 - r] = torch.tensor([1, -1, struct.unpack("<i", struct.pack("<f", float(temperature[r])))[0],
                                            seed & 0xFFFFFFFF, seed >> 32, int(draws[r]), 1, 0])
    ctx = SimpleNamespace(num_tokens=rows, num_seqs=rows, logit_rows=torch.arange(rows, dtype=torch.int32).cuda(),
                          seq_of_token=torch.arange(rows, dtype=torch.int32).cuda(),
                          seq_slots=torch.arange(rows - 1, -1, -1, dtype=torch.int32).cuda(),
                          host_seq_slots=list(range(rows - 1, -1, -1)), slot_words=words.cuda())
    got = torch.empty(rows, dtype=torch.int32, device="cuda")
    hip.sample_slots(on[0], ctx, got)
    assert torch.equal(got, want)
    after = ctx.slot_words.cpu()
    assert after[:, 1].flip(0).tolist() == want.cpu().tolist() and after[:, 5].flip(0).tolist() == (draws + 1).tolist()


def test_sampling_follows_the_distribution(hip):
    probs = torch.tensor([0.5, 0.25, 0.125, 0.125])
    rows = 4000
    logits = probs.log().repeat(rows, 1).cuda()
    out = torch.empty(rows, dtype=torch.int32, device="cuda")
    hip.sample(logits, torch.ones(rows, device="cuda"), torch.full((rows,), 11, dtype=torch.int64, device="cuda"),
               torch.arange(rows, dtype=torch.int32, device="cuda"), out)
    freq = torch.bincount(out.cpu().long(), minlength=4).float() / rows
    assert (freq - probs).abs().max() < 0.03


def test_sizes_are_refused_not_miscomputed(hip):
    from ampere_kv_engine_amd.kernels.hip import KernelError
    with pytest.raises(KernelError):
        hip.check_attention_sizes(4, 2, 24, 16)
    with pytest.raises(KernelError):
        hip.check_attention_sizes(4, 3, 32, 16)
    with pytest.raises(KernelError):
        hip.check_attention_sizes(4, 2, 512, 16)
    with pytest.raises(KernelError):
        hip.linear(torch.zeros(2, 3), torch.zeros(4, 3, device="cuda"), torch.zeros(2, 4, device="cuda"))
    with pytest.raises(KernelError):
        hip.linear(torch.zeros(2, 3, device="cuda"), torch.zeros(4, 5, device="cuda"), torch.zeros(2, 4, device="cuda"))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("history", [40, 100])
def test_attention_window_edge(hip, ref, dtype, history):
    """One key just inside the window and one just outside it both match the query far better than the rest: the
    output must be the inside key's value, and must change when the window moves by one."""
    window, dim, page = 17, 32, 8
    portions = [(history, 1)]
    pos = history                                        # the query's position; it sees keys pos - window + 1 .. pos
    inside, outside = pos - window + 1, pos - window
    for w, winner in ((window, inside), (window + 1, outside)):
        q, k_pages, v_pages, ctx, meta, keys, values = _attention_case(dtype, 2, 1, dim, page, portions, None, 41)
        table = meta.block_table[0]
        direction = torch.randn(dim, generator=torch.Generator().manual_seed(5))
        direction = direction / direction.norm() * 6.0
        for key, gain in ((inside, 1.0), (outside, 1.5)):   # the outside key wins whenever it is seen
            k_pages[int(table[key // page]), 0, key % page] = (direction * gain).to(dtype)
        q[0] = (direction.repeat(2) * 4.0).to(dtype)
        ctx.num_decode_seqs = 1
        want = torch.empty_like(q)
        ref.attention(q, k_pages, v_pages, ctx, meta, 2, 1, dim, dim ** -0.5, w, want)
        cctx, cmeta = _to_cuda(ctx, meta)
        got = torch.empty_like(q, device="cuda")
        hip.attention(q.cuda(), k_pages.cuda(), v_pages.cuda(), cctx, cmeta, 2, 1, dim, dim ** -0.5, w, got)
        torch.testing.assert_close(got.cpu().float(), want.float(), **attention_tol(dtype))
        seen_value = v_pages[int(table[winner // page]), 0, :, winner % page].float()
        torch.testing.assert_close(got.cpu().float()[0, :dim], seen_value, rtol=0.05, atol=0.05)


# ---- the device's persistent per-request state -------------------------------------------------------------------------

def _with_table_rows(ctx, meta, slots: int, seed: int):
    """The same step with its block table moved into a table of `slots` rows, request r's pages in row rows[r];
    every other row names no page (a kernel that read one would poison its result)."""
    generator = torch.Generator().manual_seed(seed)
    rows = torch.randperm(slots, generator=generator)[:ctx.num_seqs].int()
    table = torch.full((slots, meta.width), -1, dtype=torch.int32)
    table[rows.long()] = meta.block_table
    moved = SimpleNamespace(**vars(meta))
    moved.block_table, moved.rows = table, rows
    where = SimpleNamespace(**vars(ctx))
    where.host_seq_slots, where.seq_slots = rows.tolist(), rows
    return where, moved


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("portions", [[(64, 1), (17, 1), (0, 1)], [(5, 7), (63, 2), (130, 1), (0, 70)], [(1500, 1), (2, 1), (700, 1)]])
def test_attention_finds_a_request_s_pages_in_the_row_of_its_slot(hip, ref, dtype, portions):
    """Block tables that live on the device, a row per request slot: the kernels are told which row is which
    request's (`meta.rows`) and must give what they give for a table of the step's own."""
    q_heads, kv_heads, dim, page_size = 8, 2, 64, 16
    q, k_pages, v_pages, ctx, meta, _, _ = _attention_case(dtype, q_heads, kv_heads, dim, page_size, portions, None, 31)
    ctx.num_decode_seqs = sum(1 for _, n in portions if n == 1) if all(n == 1 for _, n in portions) else 0
    want = torch.empty_like(q)
    ref.attention(q, k_pages, v_pages, ctx, meta, q_heads, kv_heads, dim, dim ** -0.5, None, want)
    where, moved = _with_table_rows(ctx, meta, slots=len(portions) + 5, seed=3)
    again = torch.empty_like(q)
    ref.attention(q, k_pages, v_pages, where, moved, q_heads, kv_heads, dim, dim ** -0.5, None, again)
    assert torch.equal(again, want)                          # (the double reads the rows too)
    cctx, cmeta = _to_cuda(where, moved)
    cctx.seq_slots, cmeta.rows = where.seq_slots.cuda(), moved.rows.cuda()
    got = torch.full_like(q, float("nan"), device="cuda")
    hip.attention(q.cuda(), k_pages.cuda(), v_pages.cuda(), cctx, cmeta, q_heads, kv_heads, dim, dim ** -0.5, None, got)
    assert not torch.isnan(got).any()
    torch.testing.assert_close(got.cpu().float(), want.float(), **attention_tol(dtype))


def test_step_prologue_applies_a_step_s_changes(hip, ref):
    """(offset, value) pairs up to the count that lies on the device - never more than the capacity, never outside
    the state - and the requests' lengths into word 0 of their slots."""
    slots, width = 6, 10
    state = torch.arange(slots * 8 + slots * width, dtype=torch.int32) + 1000
    patches = torch.tensor([50, -1, 61, 7, 48, 3, 10 ** 6, 9, 55, 5, 56, 6], dtype=torch.int32)      # 6 pairs, one outside
    for count in (0, 4, 6):
        ctx = SimpleNamespace(slot_state=state.clone(), patches=patches.clone(), patch_count=torch.tensor([count], dtype=torch.int32),
                              patch_room=5, seq_slots=torch.tensor([4, 1], dtype=torch.int32),
                              seq_lens=torch.tensor([77, 9], dtype=torch.int32), num_seqs=2)
        ctx.patches = ctx.patches[:10]
        want = state.clone()
        for offset, value in list(zip(patches[0::2].tolist(), patches[1::2].tolist()))[:min(count, 5)]:
            if 0 <= offset < want.numel():
                want[offset] = value
        want[4 * 8], want[1 * 8] = 77, 9
        on = SimpleNamespace(**{k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in vars(ctx).items()})
        hip.step_prologue(on)
        assert torch.equal(on.slot_state.cpu(), want), count


def test_sampling_from_the_slots_equals_sampling_with_the_same_state_handed_in(hip, ref):
    """`sample_slots` reads temperature, seed and draw count from the slot of each row's request, chooses what `sample`
    chooses for them, and leaves the token and the next draw count in the slot; other slots are not touched."""
    import struct
    vocab, slots = 1000, 7
    logits = torch.randn(3, vocab, generator=torch.Generator().manual_seed(5)) * 3
    logits[2, 5] = float("nan")
    words = torch.full((slots, 8), 99, dtype=torch.int32)
    state = {5: (0.0, 0, 4), 2: (0.8, (1 << 40) + 12345, 7), 0: (1.5, 3, 0)}       # slot -> temperature, seed, draws
    for slot, (t, seed, draws) in state.items():
        words[slot] = torch.tensor([11, -1, struct.unpack("<i", struct.pack("<f", t))[0], seed & 0xFFFFFFFF, seed >> 32, draws, 1, 0])
    # three requests in slots 5, 2, 0; five token rows; the wanted rows are rows 4, 0 and 2
    ctx = SimpleNamespace(num_tokens=5, num_seqs=3, logit_rows=torch.tensor([4, 0, 2], dtype=torch.int32),
                          seq_of_token=torch.tensor([1, 1, 2, 2, 0], dtype=torch.int32),
                          seq_slots=torch.tensor([5, 2, 0], dtype=torch.int32), host_seq_slots=[5, 2, 0], slot_words=words.clone())
    order = [5, 2, 0]                                                             # the slots of the three logits rows
    want = torch.empty(3, dtype=torch.int32)
    ref.sample(logits, torch.tensor([state[s][0] for s in order]), torch.tensor([state[s][1] for s in order]),
               torch.tensor([state[s][2] for s in order], dtype=torch.int32), want)
    assert want[2] == -1
    on = SimpleNamespace(**{k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in vars(ctx).items()})
    got = torch.empty(3, dtype=torch.int32, device="cuda")
    hip.sample_slots(logits.cuda(), on, got)
    assert got.cpu().tolist() == want.tolist()
    after = on.slot_words.cpu()
    for row, slot in enumerate(order):
        assert after[slot, 1] == want[row] and after[slot, 5] == state[slot][2] + 1
        assert after[slot, 0] == 11 and after[slot, 2:5].tolist() == words[slot, 2:5].tolist()
    assert torch.equal(after[[1, 3, 4, 6]], words[[1, 3, 4, 6]])
    double = SimpleNamespace(**vars(ctx))
    double.slot_words = words.clone()
    chosen = torch.empty(3, dtype=torch.int32)
    ref.sample_slots(logits, double, chosen)
    assert chosen.tolist() == want.tolist() and torch.equal(double.slot_words, after)


def test_embed_takes_the_token_chosen_last_from_the_slot(hip, ref):
    table = torch.randn(50, 24, generator=torch.Generator().manual_seed(1)).bfloat16()
    words = torch.zeros(4, 8, dtype=torch.int32)
    words[3, 1], words[1, 1] = 17, 42
    ctx = SimpleNamespace(num_seqs=2, seq_of_token=torch.tensor([0, 1, 1], dtype=torch.int32),
                          seq_slots=torch.tensor([3, 1], dtype=torch.int32), host_seq_slots=[3, 1], slot_words=words)
    ids = torch.tensor([-1, 7, -1], dtype=torch.int32)
    want = table[[17, 7, 42]].float()
    out = torch.empty(3, 24)
    ref.embed(ids, table, out, ctx)
    assert torch.equal(out, want)
    on = SimpleNamespace(**{k: (v.cuda() if isinstance(v, torch.Tensor) else v) for k, v in vars(ctx).items()})
    got = torch.empty(3, 24, device="cuda")
    hip.embed(ids.cuda(), table.cuda(), got, on)
    assert torch.equal(got.cpu(), want)
    hip.embed(ids.cuda(), table.cuda(), got)                                     # without the slots -1 is no token
    assert torch.isnan(got[0]).all() and torch.equal(got[1].cpu(), want[1])


@pytest.mark.parametrize("words,blocks", [(4 * 64 * 1000, 64), (4 * 977, 7), (4 * 64 * 3 + 4 * 5, 1024), (4, 3)])
def test_read_probe_reads_every_word_once(hip, words, blocks):
    """The kernel that measures what memory gives: the xor over its per-block results is the xor of all words, whatever
    the split into blocks and waves (spans that are no whole tiles, more waves than tiles)."""
    data = torch.randint(-2 ** 31, 2 ** 31 - 1, (words,), dtype=torch.int32, generator=torch.Generator().manual_seed(3))
    want = 0
    for word in data.tolist():
        want ^= word & 0xffffffff
    got = 0
    for word in hip.read_probe(data.cuda(), blocks=blocks).cpu().tolist():
        got ^= word & 0xffffffff
    assert got == want
