"""Each HIP kernel alone against the plain torch function of the same name
(tests/emulated_ops.py), in float32 and in bfloat16, at sizes other than the
tiny models': widths and vocabularies that are no power of two, several head
sizes, group sizes and page sizes."""
import math
import random
import types

import pytest
import torch

from emulated_ops import EmulatedOps

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
# elementwise results are rounded once to the activation dtype: half an ulp
ELEM_TOL = {torch.float32: 2e-6, torch.bfloat16: 2 ** -8}


@pytest.fixture(scope="module", params=DTYPES, ids=["float32", "bfloat16"])
def both(request):
    from servelab_amd.kernels import HipOps
    dt = request.param
    return HipOps(dt, "cuda:0"), EmulatedOps(dt), dt


def randn(*shape, dtype=torch.float32, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).cuda()


def rel_err(got, ref):
    got, ref = got.float(), ref.float()
    return ((got - ref).abs().max() / ref.abs().max().clamp_min(1e-6)).item()


def test_embed(both):
    ops, emu, dt = both
    table = randn(1000, 96, dtype=dt)
    ids = torch.tensor([0, 999, 5, 5, 317], dtype=torch.int32).cuda()
    assert torch.equal(ops.embed(ids, table), emu.embed(ids, table))


@pytest.mark.parametrize("T,H", [(1, 64), (7, 3584), (33, 1000), (5, 130)])
def test_add_rmsnorm(both, T, H):
    ops, emu, dt = both
    resid = randn(T, H, seed=1)
    delta = randn(T, H, dtype=dt, seed=2)
    w = 1 + 0.1 * randn(H, seed=3)
    r1, r2 = resid.clone(), resid.clone()
    got = ops.add_rmsnorm(r1, delta, w, 1e-5)
    ref = emu.add_rmsnorm(r2, delta, w, 1e-5)
    assert (r1 - r2).abs().max().item() < 1e-6
    assert rel_err(got, ref) < ELEM_TOL[dt] * 2
    # without a delta the stream is left alone
    r3 = resid.clone()
    got = ops.add_rmsnorm(r3, None, w, 1e-6)
    assert torch.equal(r3, resid)
    assert rel_err(got, emu.add_rmsnorm(resid.clone(), None, w, 1e-6)) < ELEM_TOL[dt] * 2


def test_rows_add_rmsnorm(both):
    ops, emu, dt = both
    resid, delta = randn(20, 200, seed=1), randn(20, 200, dtype=dt, seed=2)
    w = 1 + 0.1 * randn(200, seed=3)
    rows = torch.tensor([19, 0, 7, 7], dtype=torch.int32).cuda()
    before = resid.clone()
    got = ops.rows_add_rmsnorm(resid, delta, rows, w, 1e-6)
    assert torch.equal(resid, before)
    assert rel_err(got, emu.rows_add_rmsnorm(resid, delta, rows, w, 1e-6)) < ELEM_TOL[dt] * 2
    got = ops.rows_add_rmsnorm(resid, None, rows, w, 1e-6)
    assert rel_err(got, emu.rows_add_rmsnorm(resid, None, rows, w, 1e-6)) < ELEM_TOL[dt] * 2


@pytest.mark.parametrize("T,H,ks,bias", [(20, 200, 3, True), (64, 3584, 8, False), (33, 1000, 1, True),
                                         (17, 130, 5, False)])
def test_norm_adds_partial_sums(both, T, H, ks, bias):
    """A delta given as the float partial sums of a split product (and a bias):
    the norm adds them up itself, over all rows and over chosen rows."""
    from servelab_amd.kernels.ops import PartialSums
    ops, emu, dt = both
    resid = randn(T, H, seed=1)
    parts = randn(ks, T, H, seed=2)
    b = randn(H, seed=4) if bias else None
    w = 1 + 0.1 * randn(H, seed=3)
    delta = parts.sum(0) + (b if bias else 0)
    r1, r2 = resid.clone(), resid.clone()
    got = ops.add_rmsnorm(r1, PartialSums(parts, b), w, 1e-5)
    r2 += delta
    want = (r2 * torch.rsqrt(r2.pow(2).mean(-1, keepdim=True) + 1e-5) * w).to(dt)
    assert (r1 - r2).abs().max().item() < 1e-5
    assert rel_err(got, want) < ELEM_TOL[dt] * 2
    rows = torch.tensor([T - 1, 0, 7, 7], dtype=torch.int32).cuda()
    before = resid.clone()
    got = ops.rows_add_rmsnorm(resid, PartialSums(parts, b), rows, w, 1e-5)
    assert torch.equal(resid, before)
    assert rel_err(got, want[rows.long()]) < ELEM_TOL[dt] * 2


@pytest.mark.parametrize("M,N,K", [(17, 3584, 3584), (64, 3584, 18944), (40, 132, 352), (33, 1000, 64)])
def test_deferred_product_of_many_rows(M, N, K):
    """``linear(..., defer=True)`` at 17 to 64 rows: whatever comes back (partial
    sums of a split K, or the plain product), the norm that takes it as its
    delta must see x W^T + bias."""
    from servelab_amd.kernels import HipOps
    dt = torch.bfloat16
    ops = HipOps(dt, "cuda:0")
    x, w, b = randn(M, K, dtype=dt, seed=1), (0.05 * randn(N, K, seed=2)).to(dt), randn(N, seed=3)
    weight = ops.prepare_weight(w)
    gain = 1 + 0.1 * randn(N, seed=4)
    resid = randn(M, N, seed=5)
    for bias in (None, b):
        delta = ops.linear(x, weight, bias, defer=True)
        r1 = resid.clone()
        got = ops.add_rmsnorm(r1, delta, gain, 1e-6)
        r2 = resid + x.float() @ w.float().T + (bias if bias is not None else 0)
        want = r2 * torch.rsqrt(r2.pow(2).mean(-1, keepdim=True) + 1e-6) * gain
        assert rel_err(r1, r2) < 2 ** -7
        assert rel_err(got, want) < 2 ** -6
        plain = ops.materialize(delta)
        assert rel_err(plain, x.float() @ w.float().T + (bias if bias is not None else 0)) < 2 ** -6


@pytest.mark.parametrize("M,N,K", [(1, 1000, 64), (3, 130, 200), (8, 512, 3584), (16, 96, 352),
                                   (17, 200, 136), (70, 1000, 128), (130, 352, 64)])
@pytest.mark.parametrize("bias", [False, True])
def test_linear(both, M, N, K, bias):
    ops, emu, dt = both
    x, w = randn(M, K, dtype=dt, seed=1), randn(N, K, dtype=dt, scale=0.05, seed=2)
    b = randn(N, seed=3) if bias else None
    tol = 1e-5 if dt == torch.float32 else 2 ** -7
    for out_f32 in (False, True):
        if dt == torch.bfloat16 and K % 32 == 0:
            tiled = ops.linear(x, ops.prepare_weight(w), b, out_f32=out_f32)
            assert rel_err(tiled, emu.linear(x, w, b, out_f32=out_f32)) < tol, (M, N, K, out_f32)
        got = ops.linear(x, w, b, out_f32=out_f32)
        ref = emu.linear(x, w, b, out_f32=out_f32)
        assert got.dtype == ref.dtype and got.shape == ref.shape
        assert rel_err(got, ref) < tol, (M, N, K, out_f32)


def test_library_product_pads_its_rows_harmlessly():
    """Library products of fewer than 512 rows run on a multiple of 32 rows; what
    the extra rows hold (here: NaN, left behind in the allocator's block) reaches
    no result row."""
    from servelab_amd.kernels import HipOps
    ops, emu = HipOps(torch.bfloat16, "cuda:0"), EmulatedOps(torch.bfloat16)
    assert [ops.library_rows(m) for m in (65, 96, 97, 511, 512, 700)] == [96, 96, 128, 512, 512, 700]
    x, w, b = randn(70, 128, dtype=torch.bfloat16, seed=1), randn(200, 128, dtype=torch.bfloat16, scale=0.05, seed=2), randn(200, seed=3)
    for bias in (None, b):
        junk = torch.full((96, 128), float("nan"), dtype=torch.bfloat16, device="cuda:0")
        del junk
        got = ops.linear_library(x, w, bias)
        assert got.shape == (70, 200) and got.is_contiguous() and torch.isfinite(got.float()).all()
        assert rel_err(got, emu.linear(x, w, bias)) < 2 ** -7


@pytest.mark.parametrize("M,N,K", [(1, 50, 64), (7, 1000, 3584), (16, 17, 96), (33, 200, 352), (64, 130, 1024)])
@pytest.mark.parametrize("pairs", [False, True])
def test_linear_skinny(M, N, K, pairs):
    """The matrix-core few-rows kernel alone (bfloat16): ragged M and N; one
    tile of W per workgroup (the rule's choice at these sizes) and two."""
    from servelab_amd.kernels import HipOps
    ops, emu = HipOps(torch.bfloat16, "cuda:0"), EmulatedOps(torch.bfloat16)
    if pairs:
        ops._pair_tiles = lambda M, N, K, th=16: True
    x = randn(M, K, dtype=torch.bfloat16, seed=4)
    w = randn(N, K, dtype=torch.bfloat16, scale=0.1, seed=5)
    b = randn(N, seed=6)
    weight = ops.prepare_weight(w)
    assert weight.tiled is not None and weight.tiled.numel() == -(-N // 16) * 16 * K
    for bias in (None, b):
        for out_f32 in (False, True):
            got = ops.linear_skinny(x, weight, bias, out_f32)
            assert torch.equal(got, ops.linear(x, weight, bias, out_f32))
            assert rel_err(got, emu.linear(x, w, bias, out_f32)) < (2e-5 if out_f32 else 2 ** -7)


@pytest.mark.parametrize("M,N,K", [(17, 50, 64), (33, 1000, 3584), (64, 3584, 1024), (40, 130, 352), (64, 70, 2048),
                                   (65, 144, 352), (100, 1000, 3584), (128, 4608, 1024), (127, 70, 2048),
                                   (48, 1000, 352), (80, 3000, 96), (96, 130, 352), (112, 700, 128),    # three, five, six, seven blocks of 16 rows
                                   (64, 37888, 64), (20, 40016, 96),    # so many tiles that they are spread over a whole multiple of the CUs
                                   (90, 37888, 64)])                    # ... in workgroups of eight wavefronts with six blocks of rows
def test_linear_mid(M, N, K):
    """The LDS-staged 17..128-row kernel alone: whole K and K split over up to
    16 workgroups with the separate reduction, plain and gated."""
    from servelab_amd.kernels import HipOps
    ops, emu = HipOps(torch.bfloat16, "cuda:0"), EmulatedOps(torch.bfloat16)
    x = randn(M, K, dtype=torch.bfloat16, seed=4)
    w = randn(N, K, dtype=torch.bfloat16, scale=0.1, seed=5)
    weight = ops.prepare_weight(w)
    b = randn(N, seed=6)
    ref = emu.linear(x, w, b, True)
    for ks in (1, 2, 5, 16, None):
        if ks and ks > K // 32:
            continue
        assert rel_err(ops.linear_mid(x, weight, b, out_f32=True, ks=ks), ref) < 2e-5, ks
        assert rel_err(ops.linear_mid(x, weight, None, ks=ks), emu.linear(x, w, None)) < 2 ** -7, ks
    if N % 16 == 0:
        gated = ops.linear_mid(x, weight, None, gated=True)
        assert rel_err(gated, emu.silu_mul(emu.linear(x, w, None), 8)) < 2 ** -6


@pytest.mark.parametrize("M,N,K", [(17, 50, 64), (33, 1000, 3584), (64, 3584, 1024), (40, 144, 352), (64, 80, 2048)])
def test_tiled_only_weights(M, N, K):
    """Only the tiled copy kept: few rows go straight to the matrix cores, many
    rows through the row-major scratch and the library; same results as with
    both copies (whose products in tiles over the row-major copy are switched
    off here: without that copy they are not taken; with them the results agree
    to rounding)."""
    from servelab_amd.kernels import HipOps
    ops, emu = HipOps(torch.bfloat16, "cuda:0"), EmulatedOps(torch.bfloat16)
    ops.use_block_products = False
    w = randn(N, K, dtype=torch.bfloat16, scale=0.1, seed=5)
    b = randn(N, seed=6)
    both_copies = ops.prepare_weight(w)
    ops.weight_layout = "tiled"
    tiled_only = ops.prepare_weight(w.clone())
    assert tiled_only.w is None and tiled_only.shape == (N, K)
    assert torch.equal(ops.rows_of(tiled_only), w)
    for rows in (M, 100):
        x = randn(rows, K, dtype=torch.bfloat16, seed=rows)
        assert torch.equal(ops.linear(x, tiled_only, b), ops.linear(x, both_copies, b))
        ops.use_block_products = True
        assert rel_err(ops.linear(x, both_copies, b), emu.linear(x, w, b)) < 2 ** -7
        ops.use_block_products = False
    kept = ops.prepare_weight(w, keep_rows=True)
    assert kept.w is w and kept.tiled is not None
    ops.weight_layout = "rows"
    assert ops.prepare_weight(w).tiled is None
    assert rel_err(ops.linear(randn(3, K, dtype=torch.bfloat16), ops.prepare_weight(w), b),
                   emu.linear(randn(3, K, dtype=torch.bfloat16), w, b)) < 2 ** -7


@pytest.mark.parametrize("M,N,K", [(17, 50, 64), (33, 1000, 3584), (64, 3584, 1024), (40, 130, 352), (64, 70, 2048)])
def test_linear_wide(M, N, K):
    """The 17..64-row kernel alone: ragged M and N, an odd number of tiles; and that ``linear`` takes it
    for matrices below the size from which the LDS-staged kernel takes over."""
    from servelab_amd.kernels import HipOps, Tuning
    ops = HipOps(torch.bfloat16, "cuda:0", tuning=Tuning(mid_min_elements=1 << 40, mid_min_elements_many=1 << 40))
    emu = EmulatedOps(torch.bfloat16)
    x = randn(M, K, dtype=torch.bfloat16, seed=4)
    weight = ops.prepare_weight(randn(N, K, dtype=torch.bfloat16, scale=0.1, seed=5))
    b = randn(N, seed=6)
    assert rel_err(ops.linear_wide(x, weight, b, out_f32=True), emu.linear(x, weight.w, b, True)) < 2e-5
    assert rel_err(ops.linear_wide(x, weight, None), emu.linear(x, weight.w, None)) < 2 ** -7
    assert torch.equal(ops.linear(x, weight, b), ops.linear_wide(x, weight, b))


@pytest.mark.parametrize("M,N,K", [(5, 70, 24), (64, 64, 16), (65, 129, 37)])
def test_linear_kernels_separately(both, M, N, K):
    """The tiled kernel takes any K; the few-rows kernel any K that fills
    16-byte vectors."""
    ops, emu, dt = both
    x, w = randn(M, K, dtype=dt, seed=4), randn(N, K, dtype=dt, scale=0.1, seed=5)
    b = randn(N, seed=6)
    tol = 1e-5 if dt == torch.float32 else 2 ** -7
    ref = emu.linear(x, w, b)
    assert rel_err(ops.linear_tiled(x, w, b), ref) < tol
    if K % 8 == 0:
        assert rel_err(ops.linear_rows(x, w, b), ref) < tol
    else:
        from servelab_amd.kernels import KernelError
        with pytest.raises(KernelError):
            ops.linear_rows(x, w, b)


def test_silu_mul(both):
    ops, emu, dt = both
    gu = randn(9, 2 * 353, dtype=dt, scale=3.0)
    assert rel_err(ops.silu_mul(gu), emu.silu_mul(gu)) < ELEM_TOL[dt] * 2
    gu[:, :353] = 0          # gate 0 => output 0
    assert ops.silu_mul(gu).abs().max().item() == 0


@pytest.mark.parametrize("M,I,K", [(1, 352, 128), (9, 192, 64), (40, 1000, 96), (70, 24, 32), (3, 12, 64)])
@pytest.mark.parametrize("pairs", [False, True])
def test_gated_linear(both, M, I, K, pairs):
    """gate/up GEMM + silu-multiply: the fused few-rows kernel (bfloat16, blocks
    of 8; one tile of W per workgroup and two) and the two-kernel path, against
    the plain product with separate halves."""
    ops, emu, dt = both
    if pairs:
        if dt != torch.bfloat16:
            pytest.skip("tiles of W are a matter of the bfloat16 kernels")
        from servelab_amd.kernels import HipOps
        ops = HipOps(dt, "cuda:0")
        ops._pair_tiles = lambda M, N, K, th=16: True
    x = randn(M, K, dtype=dt, seed=1)
    gate, up = randn(I, K, dtype=dt, scale=0.2, seed=2), randn(I, K, dtype=dt, scale=0.2, seed=3)
    ref = emu.silu_mul(emu.linear(x, torch.cat([gate, up]), None))
    tol = 2e-5 if dt == torch.float32 else 2 ** -6
    for block in (8, I):
        if I % block:
            continue
        w = torch.stack([gate.reshape(I // block, block, K), up.reshape(I // block, block, K)], 1)
        w = w.reshape(2 * I, K).contiguous()
        assert rel_err(ops.gated_linear(x, ops.prepare_weight(w), block), ref) < tol
        assert rel_err(ops.silu_mul(ops.linear(x, w, None), block), ref) < tol


@pytest.mark.parametrize("M,H,N2", [(1, 64, 96), (8, 3584, 4608), (16, 200 * 32, 48), (5, 96, 1000), (9, 5120, 80)])
@pytest.mark.parametrize("pairs", [False, True])
@pytest.mark.parametrize("th", [16, 14, 10, 8])
def test_fused_add_norm_around_few_rows_products(M, H, N2, pairs, th):
    """A deferred product run by the norm that adds it (stream += x W1^T, rows
    left un-normalised, sums of squares by workgroup) and the products that
    read such rows (plain with bias, gated, float output with a row gather):
    same results as product, add, norm and product one after the other; with
    one tile of W per workgroup and with two; with the first matrix in tiles
    of 16 rows and in a further copy of lower tiles (the last tile partly empty)."""
    from servelab_amd.kernels import HipOps, Tuning
    from servelab_amd.kernels.ops import Deferred, ScaledRows
    # (the fused kernels at every width, also those whose steps take the LDS-staged ones by themselves)
    ops, emu = HipOps(torch.bfloat16, "cuda:0", tuning=Tuning(fused_rows_by_width=((1 << 30, 16),))), EmulatedOps(torch.bfloat16)
    if pairs:
        ops._pair_tiles = lambda M, N, K, th=16: True
    K1 = 128 if H != 3584 else 4160       # (the long one: 224 tiles, sixteen wavefronts a workgroup)
    x = randn(M, K1, dtype=torch.bfloat16, seed=1)
    if -(-H // th) > 512:
        pytest.skip("more tiles than the readers of the stream add up sums of squares for")
    w1 = ops.prepare_weight(randn(H, K1, dtype=torch.bfloat16, scale=0.1 * (128 / K1) ** 0.5, seed=2),
                            residual_delta=th != 16, _th=th)
    assert (w1.lower is None) == (th == 16) and ops._producer_copy(w1, M)[1] == th
    gain = 1 + 0.1 * randn(H, seed=3)
    resid0 = randn(M, H, seed=4)
    eps = 1e-5
    # reference: the unfused sequence in float32 with the same roundings of inputs
    delta = x.float() @ w1.w.float().T
    stream = resid0 + delta
    normed = stream * torch.rsqrt(stream.pow(2).mean(-1, keepdim=True) + eps) * gain
    resid = resid0.clone()
    deferred = ops.linear(x, w1, None, defer=True)
    assert isinstance(deferred, Deferred)
    scaled = ops.add_rmsnorm(resid, deferred, gain, eps, fuse=True)
    assert isinstance(scaled, ScaledRows) and scaled.shape == (M, H)
    assert rel_err(resid, stream) < 1e-5
    w2 = ops.prepare_weight(randn(N2, H, dtype=torch.bfloat16, scale=0.05, seed=5))
    b2 = randn(N2, seed=6)
    ref = normed @ w2.w.float().T + b2
    assert rel_err(ops.linear(scaled, w2, b2), ref) < 2 ** -6
    assert rel_err(ops.linear(scaled, w2, b2, out_f32=True), ref) < 2 ** -7
    if N2 % 16 == 0:
        got = ops.gated_linear(scaled, w2, 8)
        assert rel_err(got, emu.silu_mul((normed @ w2.w.float().T).to(torch.bfloat16), 8)) < 2 ** -5
    # the same deferred product without a reader of scaled rows, and row-gathered for a head
    resid = resid0.clone()
    plain_rows = ops.add_rmsnorm(resid, ops.linear(x, w1, None, defer=True), gain, eps)
    assert torch.is_tensor(plain_rows) and rel_err(plain_rows, normed) < 2 ** -6
    rows = torch.tensor([M - 1, 0][:min(2, M)], dtype=torch.int32).cuda()
    resid = resid0.clone()
    picked = ops.rows_add_rmsnorm(resid, ops.linear(x, w1, None, defer=True), rows, gain, eps, fuse=True)
    assert isinstance(picked, ScaledRows) and picked.shape == (rows.shape[0], H)
    assert rel_err(ops.linear(picked, w2, None, out_f32=True), normed[rows.long()] @ w2.w.float().T) < 2 ** -7
    # more rows than the fused kernels take: the product is done (whole, or as partial sums for the norm)
    big = randn(17, K1, dtype=torch.bfloat16, seed=7)
    done = ops.linear(big, w1, None, defer=True)
    assert not isinstance(done, Deferred)
    assert rel_err(ops.materialize(done), big.float() @ w1.w.float().T) < 2 ** -7


def test_lower_tiles_for_the_products_that_add_to_the_stream():
    """Which matrices get a copy in tiles of fewer than 16 rows (sizes and CU count of the measurements), from
    how many rows of x it is read, and that the layout is what the inverse kernel undoes."""
    from servelab_amd.kernels import HipOps, Tuning
    from servelab_amd.kernels.ops import _p
    ops = HipOps(torch.bfloat16, "cuda:0")
    ops._num_cus = 256
    chosen = {N: ops.producer_tile_height(N) for N in (2048, 3072, 3584, 4096, 5120, 6400, 8192)}
    assert chosen == {2048: (8, 1), 3072: (12, 1), 3584: (16, 1), 4096: (16, 1), 5120: (10, 1), 6400: (16, 1),
                      8192: (16, 1)}
    w = randn(5120, 64, dtype=torch.bfloat16, seed=1)
    weight = ops.prepare_weight(w, residual_delta=True)
    assert weight.th == 10 and weight.lower.numel() == 5120 * 64 and weight.tiled.numel() == 5120 * 64
    assert ops._producer_copy(weight, 1) == (weight.lower, 10)
    assert ops.prepare_weight(w).lower is None                       # other matrices: tiles of 16 only
    # a smaller gain is taken with another setting, and then only from 8 rows of x on (see the rule)
    keen = HipOps(torch.bfloat16, "cuda:0", tuning=Tuning(lower_tiles_min_gain=0.05))
    keen._num_cus = 256
    assert keen.producer_tile_height(3584) == (14, 8)
    weight = keen.prepare_weight(randn(3584, 64, dtype=torch.bfloat16, seed=1), residual_delta=True)
    assert keen._producer_copy(weight, 7) == (weight.tiled, 16) and keen._producer_copy(weight, 8) == (weight.lower, 14)
    for th in (16, 14, 12, 10, 8):
        N, K = 100, 96
        w = randn(N, K, dtype=torch.bfloat16, seed=th)
        tiled = torch.full((-(-N // th) * th * K,), 7.0, dtype=torch.bfloat16, device="cuda")
        back = torch.empty(N, K, dtype=torch.bfloat16, device="cuda")
        ops._call("gemm", "sl_tile_weight", _p(w), _p(tiled), N, K, th)
        ops._call("gemm", "sl_untile_weight", _p(tiled), _p(back), N, K, th)
        assert torch.equal(back, w)
        blocks = tiled.view(-(-N // th), K // 32, 4, th, 8)              # [tile][k-step][quarter of k][row][8]
        assert torch.equal(blocks[2, 1, 3, 5], w[2 * th + 5, 32 + 24:32 + 32])
        assert not blocks[-1, :, :, N - (N // th) * th:].any() or N % th == 0   # rows beyond N are zero
    off = HipOps(torch.bfloat16, "cuda:0", tuning=Tuning(lower_tiles_min_gain=1.0))
    assert off.prepare_weight(randn(5120, 64, dtype=torch.bfloat16, seed=1), residual_delta=True).lower is None


@pytest.mark.parametrize("M,H,N2", [(1, 1536, 96), (8, 3584, 4608), (16, 5120, 1008), (5, 2048, 1000),
                                    (7, 2048, 17600), (16, 4096, 18000), (3, 5120, 16), (8, 3584, 20000)])
def test_consumer_products_on_workgroups_that_stay(M, H, N2):
    """The products that read un-normalised rows, on workgroups that keep x in registers and walk
    the tiles (several rounds where the matrix has more tiles than the chip holds workgroups):
    the very numbers of the kernel with a workgroup per tile (the same but for a last bit of the
    float32 sums at 8 rows and fewer, where that kernel loads x for two k-steps at once), which the
    test above holds to the unfused sequence.  Row lengths the kernel is not built for are refused."""
    from servelab_amd.kernels import HipOps, KernelError
    from servelab_amd.kernels.ops import ScaledRows
    ops = HipOps(torch.bfloat16, "cuda:0")
    np_ = -(-H // 16)
    assert ops._takes_resident(1 << 20, H, np_) and not ops._takes_resident(1 << 20, H + 32, np_ + 2)
    assert not ops._takes_resident(1 << 20, 8192, 512)        # measured slower there: not built
    assert not ops._takes_resident(16 * ops._num_cus, H, np_) and not ops._takes_resident(1 << 20, H, 1 << 20)
    routed = ops._takes_resident
    x = randn(M, H, dtype=torch.bfloat16, seed=1)
    parts = randn(-(-H // 16), 16, seed=2).abs().contiguous()
    w2 = ops.prepare_weight(randn(N2, H, dtype=torch.bfloat16, scale=0.05, seed=5))
    b2 = randn(N2, seed=6)
    rows = torch.tensor([M - 1, 0, M // 2][:min(3, M)], dtype=torch.int32).cuda()
    cases = [(ScaledRows(x, parts, 1e-5), b2, False), (ScaledRows(x, parts, 1e-5), None, True),
             (ScaledRows(x, parts, 1e-5, rows), None, True)]
    got = {}
    for stay in (False, True):
        ops._takes_resident = lambda N, K, parts, stay=stay: stay
        got[stay] = [ops.linear(xs, w2, b, out_f32=f32) for xs, b, f32 in cases]
        if N2 % 16 == 0:
            got[stay].append(ops.gated_linear(ScaledRows(x, parts, 1e-5), w2, 8))
    for a, b in zip(got[False], got[True]):
        assert a.shape == b.shape
        if a.shape[0] > 8:
            assert torch.equal(a, b)
        else:       # (at most 8 rows: the kernel with a workgroup per tile adds up even and odd k-steps apart)
            assert rel_err(a, b) < (2e-6 if a.dtype == torch.float32 else 2 ** -8)
            assert (a != b).float().mean() < (1.0 if a.dtype == torch.float32 else 0.02)
    # and against the formula
    inv = torch.rsqrt(parts.sum(0)[:M] / H + 1e-5)
    ref = (x.float() @ w2.w.float().T) * inv[:, None] + b2
    assert rel_err(got[True][0], ref) < 2 ** -6
    odd = ScaledRows(randn(M, H + 32, dtype=torch.bfloat16, seed=1), randn(-(-(H + 32) // 16), 16, seed=2).abs(), 1e-5)
    w_odd = ops.prepare_weight(randn(16 * 3 * ops._num_cus + 16, H + 32, dtype=torch.bfloat16, scale=0.05, seed=3))
    with pytest.raises(KernelError, match="no kernel for rows of this length"):
        ops.linear(odd, w_odd, None)
    # left to itself the kernel table sends a width the kernel is not built for to the workgroup-per-tile
    # kernel, however many tiles the matrix has
    ops._takes_resident = routed
    inv = torch.rsqrt(odd.parts.sum(0)[:M] / (H + 32) + 1e-5)
    assert rel_err(ops.linear(odd, w_odd, None, out_f32=True), (odd.x.float() @ w_odd.w.float().T) * inv[:, None]) < 2 ** -6


@pytest.mark.parametrize("M,H,I", [(2, 256, 64), (8, 3584, 18944), (16, 2048, 96), (5, 96, 160), (13, 512, 4128)])
def test_gated_mlp_keeps_few_rows_by_k_step_between_its_two_products(M, H, I):
    """gate/up and down in one call: with few rows what lies between them is laid out by k-step;
    the numbers are those of the two calls with a plain tensor between them, bit for bit, from
    plain rows and from un-normalised ones, as a finished tensor and as a product left to the norm."""
    from servelab_amd.kernels import HipOps
    from servelab_amd.kernels.ops import Deferred, ScaledRows, TiledRows
    dt = torch.bfloat16
    ops = HipOps(dt, "cuda:0")
    gu = ops.prepare_weight(randn(2 * I, H, dtype=dt, scale=0.5 / H ** 0.5, seed=1))
    down = ops.prepare_weight(randn(H, I, dtype=dt, scale=1.0 / I ** 0.5, seed=2))
    x = randn(M, H, dtype=dt, seed=3)
    parts = randn(-(-H // 16), 16, seed=4).abs().contiguous()
    gain = 1 + 0.1 * randn(H, seed=5)
    resid0 = randn(M, H, seed=6)
    got = {}
    for tiled in (False, True):
        ops.tile_few_rows = tiled
        out = []
        for xin in (x, ScaledRows(x, parts, 1e-5)):
            out.append(ops.gated_mlp(xin, gu, 8, down))
            d = ops.gated_mlp(xin, gu, 8, down, defer=True)
            assert isinstance(d, Deferred) and isinstance(d.x, TiledRows) == tiled
            if tiled:                                   # what lies between is the plain tensor, rearranged
                assert torch.equal(d.x.rows(), ops.gated_linear(xin, gu, 8))
            out.append(ops.materialize(d))
            resid = resid0.clone()
            scaled = ops.add_rmsnorm(resid, d, gain, 1e-5, fuse=True)
            assert bool(scaled.tiled) == (tiled and M > 1 and H % 32 == 0)
            out += [resid, scaled.plain_x(), scaled.parts, ops.linear(scaled, gu, None)]
        got[tiled] = out
    for a, b in zip(got[False], got[True]):
        assert a.shape == b.shape and torch.equal(a, b)
    # against the formula: gate and up rows alternate in blocks of 8
    w = gu.w.float().reshape(I // 8, 2, 8, H)
    h = (torch.nn.functional.silu(x.float() @ w[:, 0].reshape(I, H).T) * (x.float() @ w[:, 1].reshape(I, H).T)).to(dt)
    assert rel_err(got[True][0], h.float() @ down.w.float().T) < 2 ** -5


def test_rope_tables(both):
    ops, emu, dt = both
    D, theta = 48, 1e6
    inv = (1.0 / theta ** (torch.arange(0, D, 2, dtype=torch.float32) / D)).cuda()
    pos = torch.tensor([0, 1, 17, 4095, 32767], dtype=torch.int32).cuda()
    cos, sin = ops.rope_tables(pos, inv)
    # against float64 angles of the same float32 products
    ang = (pos.float()[:, None] * inv[None, :]).double()
    assert (cos.double() - torch.cos(ang)).abs().max().item() < 2e-7
    assert (sin.double() - torch.sin(ang)).abs().max().item() < 2e-7


@pytest.mark.parametrize("pairs8", [False, True])
@pytest.mark.parametrize("T", [5, 37, 400])        # per-pair kernel for few tokens, the vectorised kernel for many
@pytest.mark.parametrize("nh,nkv,D,page", [(4, 2, 16, 16), (6, 1, 48, 32), (7, 7, 128, 64), (3, 1, 24, 16)])
def test_rope_store(both, nh, nkv, D, page, pairs8, T):
    ops, emu, dt = both
    if pairs8 and D % 16:
        pytest.skip("the blocked pair order needs head sizes in steps of 16")
    pages = 9 if T < 100 else 30
    qkv = randn(T, (nh + 2 * nkv) * D, dtype=dt, seed=1)
    inv = (1.0 / 10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D)).cuda()
    pos = torch.arange(100, 100 + T, dtype=torch.int32).cuda()
    cos, sin = emu.rope_tables(pos, inv)
    slots = torch.randperm(pages * page)[:T].to(torch.int32).cuda()
    kc = [randn(pages, nkv, page, D, dtype=dt, seed=7) for _ in range(2)]
    vc = [randn(pages, nkv, D, page, dtype=dt, seed=8) for _ in range(2)]
    q1, q2 = qkv.clone(), qkv.clone()
    ops.rope_store(q1, nh, nkv, D, cos, sin, slots, kc[0], vc[0], page, pairs8)
    emu.rope_store(q2, nh, nkv, D, cos, sin, slots, kc[1], vc[1], page, pairs8)
    assert rel_err(q1, q2) < ELEM_TOL[dt] * 2
    assert rel_err(kc[0], kc[1]) < ELEM_TOL[dt] * 2
    assert torch.equal(vc[0], vc[1])
    # no tables: nothing rotates; no pages: nothing is written
    q3 = qkv.clone()
    ops.rope_store(q3, nh, nkv, D, None, None, slots, kc[0], vc[0], page)
    assert torch.equal(q3, qkv)
    k_before = kc[0].clone()
    ops.rope_store(qkv.clone(), nh, nkv, D, cos, sin, None, None, None, page)
    assert torch.equal(kc[0], k_before)


@pytest.mark.parametrize("T", [9, 400])
@pytest.mark.parametrize("nh,nkv,D,rot,page,pairs8", [(4, 2, 32, 16, 16, True), (4, 2, 32, 16, 16, False),
                                                      (6, 1, 48, 32, 32, True), (3, 3, 24, 10, 16, False),
                                                      (2, 1, 128, 64, 64, True), (5, 1, 64, 0, 16, True)])
def test_rope_store_of_a_part_of_the_head(both, nh, nkv, D, rot, page, pairs8, T):
    """Only the first ``rot`` channels of every q and k head turn (tables [T, rot / 2]); the rest
    pass, to the buffer and to the pages; rot = 0 turns nothing and still writes the pages."""
    ops, emu, dt = both
    pages = 30
    qkv = randn(T, (nh + 2 * nkv) * D, dtype=dt, seed=1)
    cos = sin = None
    if rot:
        inv = (1.0 / 10000.0 ** (torch.arange(0, rot, 2, dtype=torch.float32) / rot)).cuda()
        cos, sin = emu.rope_tables(torch.arange(100, 100 + T, dtype=torch.int32).cuda(), inv)
    slots = torch.randperm(pages * page)[:T].to(torch.int32).cuda()
    kc = [randn(pages, nkv, page, D, dtype=dt, seed=7) for _ in range(2)]
    vc = [randn(pages, nkv, D, page, dtype=dt, seed=8) for _ in range(2)]
    q1, q2 = qkv.clone(), qkv.clone()
    ops.rope_store(q1, nh, nkv, D, cos, sin, slots, kc[0], vc[0], page, pairs8, rot_dim=rot)
    emu.rope_store(q2, nh, nkv, D, cos, sin, slots, kc[1], vc[1], page, pairs8, rot_dim=rot)
    assert rel_err(q1, q2) < ELEM_TOL[dt] * 2
    assert rel_err(kc[0], kc[1]) < ELEM_TOL[dt] * 2
    assert torch.equal(vc[0], vc[1])
    heads = q1[:, :(nh + nkv) * D].view(T, nh + nkv, D)
    assert torch.equal(heads[..., rot:], qkv[:, :(nh + nkv) * D].view(T, nh + nkv, D)[..., rot:])
    with pytest.raises(Exception, match="rotate"):
        ops.rope_store(q1, nh, nkv, D, cos, sin, slots, kc[0], vc[0], page, pairs8, rot_dim=D + 2)
    # q_scale: the q heads (and nothing else) leave multiplied by it, rounded once
    q3 = qkv.clone()
    k3, v3 = kc[1].clone(), vc[1].clone()
    ops.rope_store(q3, nh, nkv, D, cos, sin, slots, k3, v3, page, pairs8, rot_dim=rot, q_scale=0.1275)
    want = q2.float()
    q_exact = qkv.float().clone()
    emu32 = EmulatedOps(torch.float32)
    emu32.rope_store(q_exact, nh, nkv, D, cos, sin, None, None, None, page, pairs8, rot_dim=rot)
    want[:, :nh * D] = (q_exact[:, :nh * D] * 0.1275).to(dt).float()
    assert rel_err(q3[:, :nh * D], want[:, :nh * D]) < ELEM_TOL[dt] * 2
    assert torch.equal(q3[:, nh * D:], q1[:, nh * D:]) and torch.equal(k3, kc[0]) and torch.equal(v3, vc[0])


def test_rotation_plans():
    """The channel order the kernel table asks a mixer for: identity when nothing turns or the
    width is no multiple of 16, blocks of 8 and partners otherwise, interleaved pairs first
    gathered into halves; a permutation in every case, the unrotated channels in place."""
    import types
    from servelab_amd.kernels import HipOps
    ops = HipOps(torch.bfloat16, "cuda:0")
    lay = lambda rot, pairing="half": types.SimpleNamespace(rot_dim=rot, pairing=pairing)
    assert ops.plan_rotation(64, None).order is None and ops.plan_rotation(64, None).rot_dim == 0
    plan = ops.plan_rotation(24, lay(10))
    assert plan.order is None and not plan.blocked and plan.rot_dim == 10
    plan = ops.plan_rotation(32, lay(32))
    assert plan.blocked and plan.order.tolist() == (list(range(0, 8)) + list(range(16, 24)) +
                                                    list(range(8, 16)) + list(range(24, 32)))
    plan = ops.plan_rotation(48, lay(16, "interleaved"))
    assert plan.order.tolist() == [0, 2, 4, 6, 8, 10, 12, 14, 1, 3, 5, 7, 9, 11, 13, 15] + list(range(16, 48))
    plan = ops.plan_rotation(16, lay(6, "interleaved"))
    assert plan.order.tolist() == [0, 2, 4, 1, 3, 5] + list(range(6, 16)) and not plan.blocked
    for bad in (lay(7), lay(40), lay(8, "quads")):
        with pytest.raises(Exception, match="no kernel"):
            ops.plan_rotation(32, bad)
    with pytest.raises(Exception, match="no kernel"):
        ops.project_qkv(None, None, None, 4, 2, 32, ops.plan_rotation(32, lay(32)), object(),
                        None, None, None, 16)


@pytest.mark.parametrize("T,nparts", [(40, 3), (400, 3), (400, 1)])
@pytest.mark.parametrize("nh,nkv,D,page", [(4, 2, 16, 16), (28, 4, 128, 16), (5, 1, 48, 32), (3, 1, 96, 64)])
def test_rope_store_from_partial_sums(both, nh, nkv, D, page, T, nparts):
    """The q/k/v product arrives as float partial sums of a split K plus a bias:
    rotation and cache write see their sum; q lands in the buffer.  With few tokens or
    several sums one block per token and head, with many tokens and one sum (the library's
    float32 product) the vectorised kernel."""
    from servelab_amd.kernels.ops import PartialSums
    ops, emu, dt = both
    pages, N = -(-T // page) + 3, (nh + 2 * nkv) * D
    parts = randn(nparts, T, N, seed=1)
    bias = randn(N, seed=2)
    inv = (1.0 / 10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D)).cuda()
    cos, sin = emu.rope_tables(torch.arange(50, 50 + T, dtype=torch.int32).cuda(), inv)
    slots = torch.randperm(pages * page)[:T].to(torch.int32).cuda()
    kc = [randn(pages, nkv, page, D, dtype=dt, seed=7) for _ in range(2)]
    vc = [randn(pages, nkv, D, page, dtype=dt, seed=8) for _ in range(2)]
    for b in (bias, None):
        for c, s_ in ((cos, sin), (None, None)):
            full = parts.sum(0) + (b if b is not None else 0)
            q1 = torch.zeros(T, N, dtype=dt, device="cuda")
            ops.rope_store(q1, nh, nkv, D, c, s_, slots, kc[0], vc[0], page, D % 16 == 0,
                           split=PartialSums(parts, b))
            q2 = full.clone()                                    # the reference rotates in float32
            EmulatedOps(torch.float32).rope_store(q2, nh, nkv, D, c, s_, slots, kc[1], vc[1], page,
                                                  D % 16 == 0)
            assert rel_err(q1[:, :nh * D], q2[:, :nh * D]) < ELEM_TOL[dt] * 2
            assert rel_err(kc[0], kc[1]) < ELEM_TOL[dt] * 2
            assert rel_err(vc[0], vc[1]) < ELEM_TOL[dt] * 2
    if dt == torch.bfloat16:
        assert rel_err(ops.materialize(PartialSums(parts, bias)), parts.sum(0) + bias) < ELEM_TOL[dt] * 2


@pytest.mark.parametrize("M", [1, 8, 16, 40])
@pytest.mark.parametrize("nh,nkv,D,page,H,rot", [(4, 2, 16, 16, 64, 16), (28, 4, 128, 16, 256, 128),
                                                 (5, 1, 48, 32, 96, 48), (5, 1, 48, 32, 96, 16),
                                                 (6, 2, 64, 16, 128, 32),
                                                 # the 7B shape's own (more tiles than CUs) and an uneven split of K
                                                 (28, 4, 128, 16, 3584, 128), (40, 8, 128, 64, 2144, 64)])
@pytest.mark.parametrize("pairs", [False, True])
def test_qkv_rope_store(M, nh, nkv, D, page, H, rot, pairs):
    """Product + rotation + cache write: the one fused kernel (at most 16 rows)
    and the product followed by rope_store give the same q, K pages and V
    pages; also with un-normalised input rows and with no rotation or no write;
    with one tile of W per workgroup and with two."""
    from servelab_amd.kernels import HipOps
    from servelab_amd.kernels.ops import ScaledRows
    dt = torch.bfloat16
    ops, emu = HipOps(dt, "cuda:0"), EmulatedOps(dt)
    if pairs:
        ops._pair_tiles = lambda M, N, K, th=16: True
    N = (nh + 2 * nkv) * D
    x = randn(M, H, dtype=dt, seed=1)
    w = ops.prepare_weight(randn(N, H, dtype=dt, scale=0.1 * min(1.0, (256 / H) ** 0.5), seed=2))
    bias = randn(N, scale=0.1, seed=3)
    inv = (1.0 / 10000.0 ** (torch.arange(0, rot, 2, dtype=torch.float32) / rot)).cuda()
    cos, sin = emu.rope_tables(torch.arange(7, 7 + M, dtype=torch.int32).cuda(), inv)
    pages = 8
    slots = torch.randperm(pages * page)[:M].to(torch.int32).cuda()

    def run(o, xin, cos, sin, write):
        kc = randn(pages, nkv, page, D, dtype=dt, seed=7)
        vc = randn(pages, nkv, D, page, dtype=dt, seed=8)
        qkv = o.qkv_rope_store(xin, w if o is ops else w.w, bias, nh, nkv, D, cos, sin,
                               slots if write else None, kc if write else None,
                               vc if write else None, page, rot_dim=rot)
        return qkv[:, :nh * D].float(), kc.float(), vc.float()
    for c, s_, write in ((cos, sin, True), (None, None, True), (cos, sin, False)):
        got, want = run(ops, x, c, s_, write), run(emu, x, c, s_, write)
        for g, r in zip(got, want):
            assert rel_err(g, r) < 2 ** -6
    if M <= 16:
        # un-normalised rows: x * gain with the sums of squares in parts
        stream = randn(M, H, seed=9)
        gain = 1 + 0.1 * randn(H, seed=10)
        parts = torch.zeros(-(-H // 16), 16, device="cuda")
        sq = stream.pow(2).view(M, -1, 16).sum(-1)                  # [M, H / 16]
        parts[:, :M] = sq.T
        scaled = ScaledRows((stream * gain).to(dt), parts, 1e-5)
        normed = (stream * torch.rsqrt(stream.pow(2).mean(-1, keepdim=True) + 1e-5) * gain).to(dt)
        got, want = run(ops, scaled, cos, sin, True), run(emu, normed, cos, sin, True)
        for g, r in zip(got, want):
            assert rel_err(g, r) < 2 ** -5


def test_a_row_gives_the_same_keys_whichever_path_its_step_takes():
    """q/k/v with a bias that bfloat16 cannot hold, for the same 300 rows in one step (library
    product) and in steps of 8 and of 40 rows (few-rows kernels): every route adds the float32
    bias to float32 sums and rounds once, so q and the cached K and V agree except where the
    order of a sum moves a value across a rounding boundary (a fraction of a per cent of the
    entries, by one step of bfloat16).  Rounding the bias to bfloat16 first, or rounding the
    product before the bias is added, changes a quarter of the entries."""
    from servelab_amd.kernels import HipOps
    dt = torch.bfloat16
    ops = HipOps(dt, "cuda:0")
    nh, nkv, D, page, H, M = 8, 2, 64, 16, 3072, 300       # (the library takes products of more than 128 rows)
    N = (nh + 2 * nkv) * D
    x = randn(M, H, dtype=dt, seed=1)
    w = ops.prepare_weight(randn(N, H, dtype=dt, scale=0.02, seed=2))
    bias = (randn(N, scale=2.0, seed=3) * 1.001).contiguous()
    assert (bias.bfloat16().float() != bias).float().mean() > 0.9
    inv = (1.0 / 10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D)).cuda()
    emu = EmulatedOps(dt)
    cos, sin = emu.rope_tables(torch.arange(M, dtype=torch.int32).cuda(), inv)
    pages = -(-M // page)
    slots = torch.randperm(pages * page)[:M].to(torch.int32).cuda()

    def run(rows_per_step):
        kc = torch.zeros(pages, nkv, page, D, dtype=dt, device="cuda")
        vc = torch.zeros(pages, nkv, D, page, dtype=dt, device="cuda")
        q = []
        for a in range(0, M, rows_per_step):
            b = min(M, a + rows_per_step)
            qkv = ops.qkv_rope_store(x[a:b].contiguous(), w, bias, nh, nkv, D, cos[a:b].contiguous(),
                                     sin[a:b].contiguous(), slots[a:b].contiguous(), kc, vc, page)
            q.append(qkv[:, :nh * D].float())
        return torch.cat(q), kc.float(), vc.float()
    assert ops._few_rows_limit(w) == 128
    whole, by8, by40 = run(M), run(8), run(40)
    for other in (by8, by40):
        for a, b in zip(whole, other):
            differ = (a != b).float().mean().item()
            assert differ < 0.01, differ
            assert ((a - b).abs() <= 2 ** -7 * a.abs().clamp_min(2 ** -6)).all()


def make_attention_case(dt, nh, nkv, D, page, seqs, seed=0):
    """``seqs``: list of (context length after the step, query length).  Builds
    a cache with shuffled pages and garbage in unused rows."""
    g = torch.Generator().manual_seed(seed)
    bs = page
    n_pages = sum(-(-c // bs) for c, _ in seqs) + 3
    perm = torch.randperm(n_pages, generator=g).tolist()
    kc = randn(n_pages, nkv, bs, D, dtype=dt, seed=seed + 1)
    vc = randn(n_pages, nkv, D, bs, dtype=dt, seed=seed + 2)
    max_pages = max(-(-c // bs) for c, _ in seqs) + 1
    tables = torch.zeros(len(seqs), max_pages, dtype=torch.int32)
    tok_seq, positions, cu = [], [], [0]
    for s, (ctx, q) in enumerate(seqs):
        n = -(-ctx // bs)
        tables[s, :n] = torch.tensor([perm.pop() for _ in range(n)], dtype=torch.int32)
        tok_seq += [s] * q
        positions += list(range(ctx - q, ctx))
        cu.append(cu[-1] + q)
    T = cu[-1]
    qkv = randn(T, (nh + 2 * nkv) * D, dtype=dt, seed=seed + 3)
    batch = types.SimpleNamespace(
        num_seqs=len(seqs), num_tokens=T,
        tok_seq=torch.tensor(tok_seq, dtype=torch.int32).cuda(),
        positions=torch.tensor(positions, dtype=torch.int32).cuda(),
        cu_q=torch.tensor(cu, dtype=torch.int32).cuda(),
        ctx_len=torch.tensor([c for c, _ in seqs], dtype=torch.int32).cuda(),
        max_ctx_len=max(c for c, _ in seqs), max_q_len=max(q for _, q in seqs),
        num_prefill_seqs=sum(1 for _, q in seqs if q > 1),
        num_prefill_tokens=sum(q for _, q in seqs if q > 1))
    return qkv, kc, vc, tables.cuda(), batch


ATTN_TOL = {torch.float32: 2e-5, torch.bfloat16: 2 ** -7}
UNITS = ["scale at the scores", "scores in units of log 2"]


def in_units(units, qkv, nh, D, scale):
    """(qkv, scale) as the attention call takes them.  "scores in units of log 2": the queries are
    multiplied by scale * log2(e) where they are made (here: before their rounding) and the call
    gets ln 2, so that scale * log2(e) is 1 for the kernel: the form the engine uses, in which
    the matrix-core kernels need no multiply-add per score."""
    if units == UNITS[0]:
        return qkv, scale
    out = qkv.clone()
    out[:, :nh * D] = (qkv[:, :nh * D].float() * (scale * math.log2(math.e))).to(qkv.dtype)
    return out, math.log(2.0)



@pytest.mark.parametrize("nh,nkv,D,page", [(4, 2, 16, 16), (8, 1, 32, 16), (7, 7, 48, 32),
                                           (28, 4, 128, 16), (6, 2, 256, 64), (5, 5, 80, 16),
                                           (40, 2, 64, 32), (3, 3, 96, 16), (66, 1, 32, 16)])
@pytest.mark.parametrize("window", [None, 16, 50])
@pytest.mark.parametrize("units", UNITS)
def test_paged_attention(both, nh, nkv, D, page, window, units):
    ops, emu, dt = both
    seqs = [(130, 130), (77, 5), (64, 64), (200, 2), (16, 1), (145, 1), (1, 1), (333, 1)]
    qkv, kc, vc, tables, batch = make_attention_case(dt, nh, nkv, D, page, seqs)
    qkv, scale = in_units(units, qkv, nh, D, 1.0 / math.sqrt(D))
    got = ops.paged_attention(qkv, nh, nkv, D, kc, vc, page, tables, batch, scale, window)
    ref = emu.paged_attention(qkv.cpu(), nh, nkv, D, kc.cpu(), vc.cpu(), page, tables.cpu(),
                              types.SimpleNamespace(**{k: (v.cpu() if torch.is_tensor(v) else v)
                                                       for k, v in vars(batch).items()}),
                              scale, window)
    assert rel_err(got.cpu(), ref) < ATTN_TOL[dt]


@pytest.mark.parametrize("nh,nkv,D,page", [(8, 1, 32, 16), (28, 4, 128, 16), (6, 2, 192, 64),
                                           (40, 2, 64, 32), (3, 3, 96, 16), (66, 1, 32, 16),
                                           (16, 8, 64, 16), (32, 16, 32, 32),     # 1, 2, 4, 8, 16 kv heads: laid out by chiplet
                                           (4, 2, 256, 16)])     # 256: no LDS form; the same calls take the other kernel
@pytest.mark.parametrize("window", [None, 16, 50])
@pytest.mark.parametrize("form", ["paired", "a tile each", "unpaired", "shares"])
@pytest.mark.parametrize("units", UNITS)
def test_prompt_attention_through_lds(nh, nkv, D, page, window, form, units):
    """The prompt kernel whose wavefronts share each block of keys through LDS,
    forced at sizes far below its crossover: portions that end inside a
    workgroup's 128 columns, that start deep in a context, and one-token rows;
    whole prompts with late and early tiles paired in a workgroup, and with a
    workgroup for every tile (what launches of two or three uneven rounds of
    pairs take); tiles cut into shares of their keys (down to one block, some
    shares empty)."""
    from servelab_amd.kernels import HipOps, Tuning
    dt = torch.bfloat16
    ops, emu = HipOps(dt, "cuda:0", tuning=Tuning(pair_prompt_tiles=form != "a tile each")), EmulatedOps(dt)
    ops.SHARED_ATTENTION_MIN_CONTEXT = ops.SHARED_ATTENTION_MIN_WAVES = 0
    if form in ("paired", "a tile each"):
        seqs = [(130, 130), (64, 64), (97, 97), (333, 333), (2, 2), (1, 1)]
    else:
        seqs = [(130, 130), (277, 45), (64, 64), (200, 2), (333, 97), (16, 1), (145, 1)]
    if form == "shares":
        ops.PROMPT_SPLIT_MIN_BLOCKS, ops.PROMPT_SPLIT_WORKGROUPS = 1, 1 << 20
    qkv, kc, vc, tables, batch = make_attention_case(dt, nh, nkv, D, page, seqs, seed=5)
    qkv, scale = in_units(units, qkv, nh, D, 1.0 / math.sqrt(D))
    got = ops.paged_attention(qkv, nh, nkv, D, kc, vc, page, tables, batch, scale, window)
    ref = emu.paged_attention(qkv.cpu(), nh, nkv, D, kc.cpu(), vc.cpu(), page, tables.cpu(),
                              types.SimpleNamespace(**{k: (v.cpu() if torch.is_tensor(v) else v)
                                                       for k, v in vars(batch).items()}),
                              scale, window)
    assert rel_err(got.cpu(), ref) < ATTN_TOL[dt]


def test_portions_deep_in_a_context_take_shares_of_their_keys_by_default():
    """The launches the table chooses by itself (no threshold moved): whole prompts, short or long,
    take the kernel that shares keys through LDS with a workgroup for every tile; a portion that
    starts deep in its context, down to two tokens, has its tiles cut into shares of their keys
    (no share of fewer than 8 key blocks, none for a context of fewer than 16).  Results against
    the plain computation."""
    from servelab_amd.kernels import HipOps
    dt = torch.bfloat16
    nh, nkv, D, page = 8, 2, 64, 16
    for seqs, shares in (([(40, 40), (300, 300), (7, 7)], 1), ([(2000, 40), (700, 3), (333, 2)], 7),
                         ([(4100, 2)], 16), ([(300, 5)], 1), ([(520, 9), (514, 2)], 2)):
        ops, emu = HipOps(dt, "cuda:0"), EmulatedOps(dt)
        seen = []
        call = ops._call

        def spy(stem, name, *args):
            if name.startswith("sl_attention_mfma@"):
                seen.append((args[17], args[18], args[19]))          # shares, wavefronts for the LDS form, pairs
            return call(stem, name, *args)
        ops._call = spy
        qkv, kc, vc, tables, batch = make_attention_case(dt, nh, nkv, D, page, seqs, seed=11)
        qkv, scale = in_units(UNITS[1], qkv, nh, D, 1.0 / math.sqrt(D))
        got = ops.paged_attention(qkv, nh, nkv, D, kc, vc, page, tables, batch, scale, None)
        assert seen == [(shares, 0, 0)], (seqs, seen)
        ref = emu.paged_attention(qkv.cpu(), nh, nkv, D, kc.cpu(), vc.cpu(), page, tables.cpu(),
                                  types.SimpleNamespace(**{k: (v.cpu() if torch.is_tensor(v) else v)
                                                           for k, v in vars(batch).items()}),
                                  scale, None)
        assert rel_err(got.cpu(), ref) < ATTN_TOL[dt]


@pytest.mark.parametrize("seed", range(10))
def test_attention_over_random_batches(seed):
    """Seeded random batches through the launches the table chooses by itself: whole prompts, portions
    deep in their contexts (two tokens to hundreds), single tokens after them; 1 to 16 kv heads (laid
    out by chiplet or not), with and without a window; on a table that believes in 8 CUs, so that a few
    single tokens already merge inside their workgroups or, for every third seed, take shares of one
    length.  Against the plain computation."""
    import random
    from servelab_amd.kernels import HipOps
    rnd = random.Random(seed)
    dt = torch.bfloat16
    nkv = rnd.choice([1, 2, 3, 4, 8, 16])
    g = rnd.choice([1, 2, 7, 8, 20])
    D, page = rnd.choice([(32, 16), (64, 32), (128, 16), (96, 64)])
    nh = nkv * g
    window = rnd.choice([None, None, 40, 300])
    prompts = []
    for _ in range(rnd.randint(0, 4)):
        q = rnd.choice([2, 3, 17, 64, 130, 300])
        prompts.append((q + rnd.choice([0, 0, 5, 200, 900]), q))
    singles = [(rnd.randint(1, 1500), 1) for _ in range(rnd.choice([0, 1, 3, 9]))]
    seqs = prompts + singles or [(77, 77)]
    from servelab_amd.kernels import Tuning
    ops, emu = HipOps(dt, "cuda:0", tuning=Tuning(shares_of_one_length=seed % 3 == 0)), EmulatedOps(dt)
    ops._num_cus = 8
    qkv, kc, vc, tables, batch = make_attention_case(dt, nh, nkv, D, page, seqs, seed=seed)
    qkv, scale = in_units(UNITS[seed % 2], qkv, nh, D, 1.0 / math.sqrt(D))
    ref = emu.paged_attention(qkv.cpu(), nh, nkv, D, kc.cpu(), vc.cpu(), page, tables.cpu(),
                              types.SimpleNamespace(**{k: (v.cpu() if torch.is_tensor(v) else v)
                                                       for k, v in vars(batch).items()}),
                              scale, window)
    # (what the engine's batches say of their single tokens: the sum and the largest of their contexts)
    batch.ctx_stats = torch.tensor([sum(c for c, _ in singles), max([c for c, _ in singles] or [0])],
                                   dtype=torch.int32, device="cuda")
    got = ops.paged_attention(qkv, nh, nkv, D, kc, vc, page, tables, batch, scale, window)
    assert rel_err(got.cpu(), ref) < ATTN_TOL[dt], (nh, nkv, D, page, window, seqs)


def test_decode_shares_by_the_estimate_of_the_launch():
    """The number of shares of a request's keys at sizes it was measured at (4 kv heads, head size 128, 256
    CUs): never slightly more wavefronts than a whole number per CU where the stream of keys decides; one
    trip to memory a share where the context is short; no more shares than the combine kernel's batches
    are worth for one request with a long context."""
    from servelab_amd.kernels import HipOps
    ops = HipOps(torch.bfloat16, "cuda:0")
    ops._num_cus = 256
    at = lambda requests, ctx: ops._decode_shares(4 * requests, min(256, max(1, ctx // 64)), -(-ctx // 32), 128)
    assert {b: at(b, 4096) for b in (1, 2, 4, 8, 14, 16, 24, 48, 64)} == \
        {1: 64, 2: 32, 4: 32, 8: 16, 14: 9, 16: 8, 24: 8, 48: 4, 64: 2}
    assert {b: at(b, 1024) for b in (1, 5, 7, 8, 12, 16)} == {1: 16, 5: 16, 7: 16, 8: 16, 12: 10, 16: 8}
    assert {c: at(1, c) for c in (2048, 8192, 16384, 32768)} == {2048: 32, 8192: 64, 16384: 64, 32768: 128}
    assert ops._decode_shares(4, 1, 128, 128) == 1 and ops._decode_shares(256, 64, 128, 128) == 2
    for requests in range(1, 65):
        waves = 4 * requests * at(requests, 4096)
        assert waves <= 256 or (waves - 1) % 256 >= 128, (requests, waves)      # (no round of the CUs less than half full)


def test_whole_prompts_pair_their_tiles_unless_the_rounds_are_uneven():
    """The choice between a late tile with its early mirror per workgroup and a workgroup per tile, at the
    sizes it was measured at (7B shape: 7 columns a token, 4 kv heads, 256 CUs)."""
    from servelab_amd.kernels import HipOps
    ops = HipOps(torch.bfloat16, "cuda:0")
    ops._num_cus = 256
    paired = {T: ops._pair_prompt_tiles(-(-T * 7 // 128), 4) for T in (2048, 4096, 4608, 5120, 8192, 14336, 32768)}
    assert paired == {2048: True, 4096: True, 4608: True, 5120: False, 8192: False, 14336: False, 32768: True}
    assert ops._pair_prompt_tiles(-(-4096 * 7 // 128), 4 * 8)          # eight prompts of 4,096: seven full rounds
    ops.PAIR_PROMPT_TILES = False
    assert not ops._pair_prompt_tiles(10, 4)


@pytest.mark.parametrize("units", UNITS)
def test_attention_reference_point_moves_late(units):
    """Scores that keep growing along the context, by more than the kernels'
    lazy-rescale margin from block to block: the running reference of every
    column has to move many times, in prompt portions and in split decode."""
    from servelab_amd.kernels import HipOps
    dt = torch.bfloat16
    nh, nkv, D, page = 4, 2, 64, 16
    emu = EmulatedOps(dt)
    seqs = [(400, 400), (300, 1)]
    for shared in (0, 1 << 30):
        ops = HipOps(dt, "cuda:0")
        ops.SHARED_ATTENTION_MIN_CONTEXT = ops.SHARED_ATTENTION_MIN_WAVES = shared
        qkv, kc, vc, tables, batch = make_attention_case(dt, nh, nkv, D, page, seqs, seed=11)
        # key at position r has r / 2 on channel 0, queries have 1 there: the
        # score grows by 16 (23 in units of log 2) per block of 32 keys
        qkv[:, 0:nh * D:D] = 1.0
        for s, (ctx, _) in enumerate(seqs):
            for r in range(ctx):
                kc[int(tables[s, r // page]), :, r % page, 0] = r / 2
        qkv, scale = in_units(units, qkv, nh, D, 1.0)
        got = ops.paged_attention(qkv, nh, nkv, D, kc, vc, page, tables, batch, scale, None)
        ref = emu.paged_attention(qkv.cpu(), nh, nkv, D, kc.cpu(), vc.cpu(), page, tables.cpu(),
                                  types.SimpleNamespace(**{k: (v.cpu() if torch.is_tensor(v) else v)
                                                           for k, v in vars(batch).items()}),
                                  scale, None)
        assert rel_err(got.cpu(), ref) < ATTN_TOL[dt]


@pytest.mark.parametrize("nh,nkv,D,page", [(4, 2, 16, 16), (7, 7, 48, 32), (5, 5, 80, 16), (28, 4, 128, 16)])
@pytest.mark.parametrize("window", [None, 50])
@pytest.mark.parametrize("units", UNITS)
def test_decode_attention_shares_out_the_keys(both, nh, nkv, D, page, window, units):
    """Single-token rows only: the general kernel (float32, and bfloat16 head
    sizes the matrix-core kernels refuse) and the matrix-core kernel both split
    every row's keys over several wavefronts and merge the shares; contexts of
    1 token, of less than a share each, and of hundreds."""
    ops, emu, dt = both
    seqs = [(1, 1), (5, 1), (64, 1), (65, 1), (333, 1), (700, 1), (129, 1)]
    qkv, kc, vc, tables, batch = make_attention_case(dt, nh, nkv, D, page, seqs, seed=9)
    qkv, scale = in_units(units, qkv, nh, D, 1.0 / math.sqrt(D))
    got = ops.paged_attention(qkv, nh, nkv, D, kc, vc, page, tables, batch, scale, window)
    ref = emu.paged_attention(qkv.cpu(), nh, nkv, D, kc.cpu(), vc.cpu(), page, tables.cpu(),
                              types.SimpleNamespace(**{k: (v.cpu() if torch.is_tensor(v) else v)
                                                       for k, v in vars(batch).items()}),
                              scale, window)
    assert rel_err(got.cpu(), ref) < ATTN_TOL[dt]


@pytest.mark.parametrize("nh,nkv,D,page", [(28, 4, 128, 16), (8, 8, 32, 32), (40, 2, 64, 16), (32, 1, 96, 64), (6, 2, 256, 16)])
@pytest.mark.parametrize("window", [None, 50])
@pytest.mark.parametrize("units", UNITS)
def test_decode_attention_merged_inside_the_workgroup(nh, nkv, D, page, window, units):
    """Single-token rows with a workgroup of eight wavefronts per (request, kv head) that cut the keys
    among themselves and merge in LDS (forced here at a batch far smaller than the one that takes it
    by itself): contexts of 1 token (seven wavefronts without a key), of fewer blocks than wavefronts,
    of hundreds and of thousands of keys; 1, 7, 20 and 32 query heads a kv head (one and two column
    tiles); and that the table takes this form by itself once the batch fills the chip with it."""
    from servelab_amd.kernels import HipOps, Tuning
    dt = torch.bfloat16
    ops, emu = HipOps(dt, "cuda:0", tuning=Tuning(group_attention_fill=0.0)), EmulatedOps(dt)
    seen = []
    call = ops._call

    def spy(stem, name, *args):
        if name.startswith("sl_attention_mfma@"):
            seen.append((args[17], args[-3]))                    # shares, merged inside the workgroup
        return call(stem, name, *args)
    ops._call = spy
    seqs = [(1, 1), (5, 1), (64, 1), (65, 1), (333, 1), (700, 1), (129, 1), (4100, 1)]
    qkv, kc, vc, tables, batch = make_attention_case(dt, nh, nkv, D, page, seqs, seed=9)
    qkv, scale = in_units(units, qkv, nh, D, 1.0 / math.sqrt(D))
    got = ops.paged_attention(qkv, nh, nkv, D, kc, vc, page, tables, batch, scale, window)
    assert len(seen) == 1 and seen[0] == (1, 1)
    ref = emu.paged_attention(qkv.cpu(), nh, nkv, D, kc.cpu(), vc.cpu(), page, tables.cpu(),
                              types.SimpleNamespace(**{k: (v.cpu() if torch.is_tensor(v) else v)
                                                       for k, v in vars(batch).items()}),
                              scale, window)
    assert rel_err(got.cpu(), ref) < ATTN_TOL[dt]
    # by itself: with a pair for nearly every CU (here: a table told that it has 24 CUs), or fewer of shorter contexts
    # (0.97 of the CUs up to 4,096 keys, 0.7 up to 1,024, 0.45 up to 512, one pair up to 256; never beyond 4,096 with no more pairs than CUs)
    plain = HipOps(dt, "cuda:0")
    plain._num_cus = 24
    for n_seqs, ctx, merged in ((-(-24 // nkv), 4000, True), (max(1, 23 // nkv), 4000, False), (-(-24 // nkv), 5000, False),
                                (-(-17 // nkv), 900, True), (max(1, 16 // nkv), 900, False),
                                (-(-11 // nkv), 500, True), (max(1, 10 // nkv), 500, False),
                                (1, 200, True), (1, 300, False)) if window is None else ():      # (a window makes every context short)
        seen.clear()
        plain._call = lambda stem, name, *args: (seen.append((args[17], args[-3])) if name.startswith("sl_attention_mfma@") else None,
                                                 HipOps._call(plain, stem, name, *args))[1]
        case = make_attention_case(dt, nh, nkv, D, page, [(ctx - 3 * i, 1) for i in range(n_seqs)], seed=3)
        q2, s2 = in_units(units, case[0], nh, D, 1.0 / math.sqrt(D))
        plain.paged_attention(q2, nh, nkv, D, case[1], case[2], page, case[3], case[4], s2, window)
        assert len(seen) == 1 and bool(seen[0][1]) == bool(merged) and (seen[0][0] == 1 or not merged), (n_seqs, ctx, seen)


@pytest.mark.parametrize("nh,nkv,D,page,window", [(28, 4, 128, 16, None), (8, 1, 64, 32, None), (40, 8, 128, 16, 700), (20, 1, 128, 64, None)])
def test_single_tokens_in_shares_of_one_length(nh, nkv, D, page, window):
    """Contexts of very different lengths in one step that says how long they are: every share of the
    launch has about as many key blocks, a long sequence is cut into more shares than the plan for
    equal contexts has, a short one into one, and the wavefronts of the shares a sequence does not
    use leave a mark that the combine kernel skips.  Against the plain result, and the launch itself:
    more share slots than the plan's shares, and the step's sums on the device."""
    from servelab_amd.kernels import HipOps, Tuning
    dt = torch.bfloat16
    emu = EmulatedOps(dt)
    rng = random.Random(nh)
    told = 0
    for lens in ([4100] + [rng.randrange(1, 300) for _ in range(23)], [rng.randrange(1, 2000) for _ in range(40)],
                 [3000] * 12, [1], [5, 4100, 70, 33, 64, 65]):
        seqs = [(c, 1) for c in lens]
        qkv, kc, vc, tables, batch = make_attention_case(dt, nh, nkv, D, page, seqs, seed=len(lens))
        host = types.SimpleNamespace(**{k: (v.cpu() if torch.is_tensor(v) else v) for k, v in vars(batch).items()})
        q2, scale = in_units(UNITS[1], qkv, nh, D, 1.0 / math.sqrt(D))
        ref = emu.paged_attention(q2.cpu(), nh, nkv, D, kc.cpu(), vc.cpu(), page, tables.cpu(), host, scale, window)
        batch.ctx_stats = torch.tensor([sum(lens), max(lens)], dtype=torch.int32, device="cuda")
        for tuning in (Tuning(shares_of_one_length=True), Tuning(shares_of_one_length=True, share_slots_growth=1),
                       Tuning(shares_of_one_length=True, share_slots_growth=16, share_slots_waves=1 << 20)):
            ops = HipOps(dt, "cuda:0", tuning=tuning)
            ops._num_cus = 8                      # (more pairs than CUs from three sequences on)
            seen = []
            call = ops._call
            ops._call = lambda stem, name, *args: (seen.append(args) if name.startswith("sl_attention_mfma@") else None,
                                                   call(stem, name, *args))[1]
            got = ops.paged_attention(q2, nh, nkv, D, kc, vc, page, tables, batch, scale, window)
            assert rel_err(got.cpu(), ref) < ATTN_TOL[dt], (lens[:3], tuning.share_slots_growth)
            if len(lens) * nkv > 8 and len(seen) == 1 and seen[0][17] > 1:
                # one launch in shares: it is told the step's sums and the wavefronts to aim at
                slots, merged, stats, aim = seen[0][17], seen[0][-3], seen[0][-2], seen[0][-1]
                assert not merged and stats.value == batch.ctx_stats.data_ptr()
                assert aim % (len(lens) * nkv) == 0 and aim // (len(lens) * nkv) <= slots
                assert slots <= max(aim // (len(lens) * nkv), tuning.share_slots_growth * aim // (len(lens) * nkv))
                told += 1
        # without the step's sums: as many shares for every sequence
        del batch.ctx_stats
        ops = HipOps(dt, "cuda:0", tuning=Tuning(group_attention_fill=1e9))
        assert rel_err(ops.paged_attention(q2, nh, nkv, D, kc, vc, page, tables, batch, scale, window).cpu(), ref) < ATTN_TOL[dt]
    assert told >= 6


def test_single_tokens_of_more_pairs_than_cus():
    """More (request, kv head) pairs than CUs: the form is taken by the estimate of the launch's time
    (on a table told that it has 256 CUs: shares that fill whole rounds of the CUs between one pair a
    CU and two, merged in the workgroup where two rounds are nearly full and the context is short, one
    share once there are four wavefronts for every CU), and every form gives the plain result
    (a table told that it has 8 CUs; 4, 5, 40 and 9 requests of 4 kv heads: merged, two shares, one share,
    and two launches: eight requests, which fill whole rounds, merged and the ninth in 4 shares)."""
    from servelab_amd.kernels import HipOps
    dt = torch.bfloat16
    ops, emu = HipOps(dt, "cuda:0"), EmulatedOps(dt)
    ops._num_cus = 256
    plan = lambda pairs, blocks, fits=True: ops._decode_many(pairs, blocks, 128, fits, min(256, blocks // 2))[:2]
    assert [plan(p, 128) for p in (288, 384, 416, 576, 640, 1024, 4096)] == \
        [(False, 4), (False, 2), (False, 3), (False, 3), (False, 2), (False, 1), (False, 1)]
    assert plan(448, 32) == (True, 1) and plan(448, 32, fits=False) == (False, 2)
    assert plan(300, 2) == (True, 1) and plan(300, 2, fits=False) == (False, 1)      # (no block to share out)
    nh, nkv, D, page = 28, 4, 128, 16
    ops._num_cus = 8
    seen = []
    call = ops._call
    ops._call = lambda stem, name, *args: (seen.append((args[17], args[-3])) if name.startswith("sl_attention_mfma@") else None,
                                           call(stem, name, *args))[1]
    for n_seqs, ctx, form in ((4, 700, [(1, 1)]), (5, 3000, [(2, 0)]), (40, 700, [(1, 0)]), (9, 3000, [(1, 1), (4, 0)])):
        seqs = [(ctx - 13 * i, 1) for i in range(n_seqs)]
        qkv, kc, vc, tables, batch = make_attention_case(dt, nh, nkv, D, page, seqs, seed=ctx)
        qkv, scale = in_units(UNITS[1], qkv, nh, D, 1.0 / math.sqrt(D))
        for shares in (None, 3):                     # the form it takes by itself, and three shares
            if shares:
                ops._decode_many = lambda *a: (False, shares, 0.0)
            seen.clear()
            got = ops.paged_attention(qkv, nh, nkv, D, kc, vc, page, tables, batch, scale, None)
            assert seen == (form if shares is None else [(3, 0)]), (n_seqs, ctx, seen)
            ref = emu.paged_attention(qkv.cpu(), nh, nkv, D, kc.cpu(), vc.cpu(), page, tables.cpu(),
                                      types.SimpleNamespace(**{k: (v.cpu() if torch.is_tensor(v) else v)
                                                               for k, v in vars(batch).items()}), scale, None)
            assert rel_err(got.cpu(), ref) < ATTN_TOL[dt]
        del ops._decode_many


@pytest.mark.parametrize("nh,nkv,D,page", [(28, 4, 128, 16), (8, 1, 64, 32)])
@pytest.mark.parametrize("contexts", [(9000,), (9000, 5000)])
def test_decode_attention_with_more_shares_than_lanes(nh, nkv, D, page, contexts):
    """One or two requests with long contexts are cut into more than 64 shares (up to 141 here, with a
    launch whose estimate counts nothing but the trips to memory), of which a lane of the
    merging wavefront takes several; the key that carries the weight of request 0 lies in a late share."""
    from servelab_amd.kernels import HipOps, Tuning
    dt = torch.bfloat16
    ops, emu = HipOps(dt, "cuda:0", tuning=Tuning(few_wave_us=0.0, few_batch_us=0.0, few_stream_gbs_per_cu=1e9)), EmulatedOps(dt)
    blocks = -(-max(contexts) // 32)
    assert 64 < ops._decode_shares(len(contexts) * nkv, min(256, blocks // 2), blocks, D) <= 141
    seqs = [(c, 1) for c in contexts]
    qkv, kc, vc, tables, batch = make_attention_case(dt, nh, nkv, D, page, seqs, seed=21)
    at = 8000
    kc[int(tables[0, at // page]), :, at % page] = 4 * qkv[0, :D].float().sign().to(dt)     # head 0's query picks it
    qkv, scale = in_units(UNITS[1], qkv, nh, D, 1.0 / math.sqrt(D))
    got = ops.paged_attention(qkv, nh, nkv, D, kc, vc, page, tables, batch, scale, None)
    ref = emu.paged_attention(qkv.cpu(), nh, nkv, D, kc.cpu(), vc.cpu(), page, tables.cpu(),
                              types.SimpleNamespace(**{k: (v.cpu() if torch.is_tensor(v) else v)
                                                       for k, v in vars(batch).items()}), scale, None)
    assert rel_err(got.cpu(), ref) < ATTN_TOL[dt]
    picked = vc[int(tables[0, at // page]), 0, :, at % page].float()
    assert (got[0, :D].float() - picked).abs().max() < 0.05 * picked.abs().max()


@pytest.mark.parametrize("nh,nkv,D,page", [(4, 2, 32, 16), (28, 4, 128, 16), (6, 3, 64, 64), (5, 5, 96, 32)])
@pytest.mark.parametrize("contexts", [(700, 333, 5, 64, 65, 1, 129), (3, 2), (40,) * 16, (2000, 7, 300)])
def test_attention_and_its_projection_in_one_call(nh, nkv, D, page, contexts):
    """A step of a few single tokens through attend_and_project: what lies between the attention
    and the output projection is laid out by k-step (split contexts merged by the combine kernel,
    short ones written by the attention kernel itself); the result is that of the two calls with a
    plain tensor between them, bit for bit, finished or left to the norm."""
    from servelab_amd.kernels import HipOps
    from servelab_amd.kernels.ops import Deferred, TiledRows
    dt = torch.bfloat16
    ops = HipOps(dt, "cuda:0")
    seqs = [(c, 1) for c in contexts]
    qkv, kc, vc, tables, batch = make_attention_case(dt, nh, nkv, D, page, seqs, seed=11)
    T, H = len(seqs), 160
    w_o = ops.prepare_weight(randn(H, nh * D, dtype=dt, scale=1.0 / (nh * D) ** 0.5, seed=12))
    gain = 1 + 0.1 * randn(H, seed=13)
    resid0 = randn(T, H, seed=14)
    args = (qkv, nh, nkv, D, kc, vc, page, tables, batch, 1.0 / math.sqrt(D), None)
    plain = ops.paged_attention(*args)
    got = {}
    for tiled in (False, True):
        ops.tile_few_rows = tiled
        d = ops.attend_and_project(*args, w_o, None, defer=True)
        assert isinstance(d, Deferred) and isinstance(d.x, TiledRows) == tiled
        if tiled:
            assert torch.equal(d.x.rows(), plain)
        resid = resid0.clone()
        scaled = ops.add_rmsnorm(resid, d, gain, 1e-5, fuse=True)
        got[tiled] = [ops.attend_and_project(*args, w_o, None), ops.materialize(d), resid, scaled.plain_x()]
    for a, b in zip(got[False], got[True]):
        assert torch.equal(a, b)
    assert rel_err(got[True][0], plain.float() @ w_o.w.float().T) < 2 ** -6


@pytest.mark.parametrize("D,page", [(16, 16), (32, 16), (128, 32)])
@pytest.mark.parametrize("q_len", [1, 5])
@pytest.mark.parametrize("units", UNITS)
def test_attention_finds_one_key_at_edges(both, D, page, q_len, units):
    """One key among hundreds carries all the weight (its score stands out by
    construction), placed at a page's last and first slot, at the first and the
    last visible position, and just inside and just outside a window: the
    output must be that key's value, or must not be."""
    ops, emu, dt = both
    nh, nkv, ctx, W = 4, 2, 300, 48
    p_last = ctx - 1                                   # position of the last query
    targets = [0, page - 1, page, 2 * page - 1, 5 * page, p_last - W + 1, p_last - W, p_last]
    for window in (None, W):
        for target in targets:
            qkv, kc, vc, tables, batch = make_attention_case(dt, nh, nkv, D, page, [(ctx, q_len)], seed=3)
            qkv[:, :nh * D] = 0
            qkv[:, 0:nh * D:D] = 30.0                  # every head's query: 30 on channel 0
            kc[:, :, :, 0] = 0
            pg, off = int(tables[0, target // page]), target % page
            kc[pg, :, off, 0] = 30.0                   # score 900 for the target, 0 elsewhere
            qkv, scale = in_units(units, qkv, nh, D, 1.0)
            got = ops.paged_attention(qkv, nh, nkv, D, kc, vc, page, tables, batch, scale, window)
            last = got[-1].float().view(nh, D)         # the query at position ctx - 1
            visible = window is None or target > p_last - window
            for h in range(nh):
                hit = (last[h] - vc[pg, h // 2, :, off].float()).abs().max().item() < 2e-2
                assert hit == visible, (window, target, h)
            if q_len > 1 and target == p_last:         # earlier queries of the portion do not see it
                first = got[0].float().view(nh, D)
                assert (first[0] - vc[pg, 0, :, off].float()).abs().max().item() > 0.1


def test_argmax_and_sampling():
    from servelab_amd.kernels import HipOps
    ops = HipOps(torch.float32, "cuda:0")
    V = 152064 // 8 + 7
    logits = randn(5, V, seed=1)
    logits[2, 77] = 50.0
    logits[2, 9000] = 50.0            # ties resolve to the first index
    assert ops.argmax(logits).tolist() == torch.argmax(logits, -1).tolist()
    assert ops.argmax(logits)[2].item() == 77

    # temperature sampling follows softmax(logits / T)
    V, n = 11, 20000
    base = torch.tensor([2.0, 1.0, 0.5, 0.0, -1.0, 3.0, 0.1, 0.2, -3.0, 1.5, 2.5])
    logits = base.repeat(n, 1).cuda()
    T = 0.7
    temp = torch.full((n,), T).cuda()
    top_k = torch.full((n,), -1, dtype=torch.int32).cuda()
    top_p = torch.ones(n).cuda()
    seeds = torch.full((n,), 1234, dtype=torch.int64).cuda()
    draws = torch.arange(n, dtype=torch.int64).cuda()
    toks = ops.sample(logits, temp, top_k, top_p, seeds, draws)
    # rows without a cut draw the same token from the two-stage kernel (no top_k / top_p given)
    assert torch.equal(toks, ops.sample(logits, temp, None, None, seeds, draws))
    freq = torch.bincount(toks.long().cpu(), minlength=V).float() / n
    want = torch.softmax(base / T, -1)
    assert (freq - want).abs().max().item() < 0.015
    # same seed and draw => same token; temperature 0 rows take the argmax
    assert torch.equal(toks, ops.sample(logits, temp, top_k, top_p, seeds, draws))
    temp0 = torch.zeros(n).cuda()
    assert set(ops.sample(logits, temp0, top_k, top_p, seeds, draws).tolist()) == {5}
    # top-k 3 draws only the three largest, renormalised
    k3 = torch.full((n,), 3, dtype=torch.int32).cuda()
    toks = ops.sample(logits, temp, k3, top_p, seeds, draws)
    freq = torch.bincount(toks.long().cpu(), minlength=V).float() / n
    keep = torch.zeros(V)
    keep[[5, 10, 0]] = 1
    want3 = torch.softmax(base / T, -1) * keep
    want3 /= want3.sum()
    assert (freq - want3).abs().max().item() < 0.015
    # top-p: sorted prefix with cumulative probability <= p (first always kept)
    p = 0.8
    probs = torch.softmax(base / T, -1)
    sp, si = torch.sort(probs, descending=True)
    kept = si[(torch.cumsum(sp, 0) <= p) | (torch.arange(V) == 0)]
    wantp = torch.zeros(V)
    wantp[kept] = probs[kept]
    wantp /= wantp.sum()
    toks = ops.sample(logits, temp, top_k, torch.full((n,), p).cuda(), seeds, draws)
    freq = torch.bincount(toks.long().cpu(), minlength=V).float() / n
    assert (freq - wantp).abs().max().item() < 0.015


def assert_plain_draws(tokens, logits, temperature, top_k, top_p, seeds, draws, slack=2e-3):
    """Every token is the plain Gumbel-max draw of its row (tests/emulated_ops.py: the same
    counter-based uniforms, logarithms in float64), or ties with it within ``slack`` (the kernels
    take their logarithms from the hardware's log2)."""
    from emulated_ops import kept_by_cut, perturbed_scores
    import numpy as np
    for r, tok in enumerate(tokens.tolist()):
        T = float(temperature[r])
        if T == 0.0:
            assert tok == int(logits[r].argmax()), f"row {r}"
            continue
        scores = perturbed_scores(logits[r], T, int(seeds[r]), int(draws[r]))
        keep = kept_by_cut(logits[r], T, int(top_k[r]) if top_k is not None else -1,
                           float(top_p[r]) if top_p is not None else 1.0)
        assert keep[tok], f"row {r}: token {tok} lies outside the cut"
        best = np.where(keep, scores, -np.inf).max()
        assert scores[tok] >= best - slack, f"row {r}: token {tok} scores {scores[tok]}, best {best}"


def test_draws_are_the_plain_gumbel_draws():
    """Seeded draws over a wide row equal the plain ones, with and without cuts; the uniform that
    the hash maps to its largest value (seed 1234, draw 1, index 58452: 1 - 2^-24) stays below 1,
    so its Gumbel value is finite and a logit of -20 there is not drawn."""
    from emulated_ops import uniform01
    from servelab_amd.kernels import HipOps
    ops = HipOps(torch.float32, "cuda:0")
    R, V = 12, 152064
    assert uniform01(1234, 1, V)[58452] == 1 - 2.0 ** -24 and uniform01(1234, 1, V).max() < 1.0
    logits = 2.0 * randn(R, V, seed=17)
    logits[0] = 0.0
    logits[0, 58452] = -20.0
    temp = torch.full((R,), 0.9).cuda()
    temp[0], temp[5] = 1.0, 0.0
    seeds = (torch.arange(R, dtype=torch.int64) * 977 + 3).cuda()
    draws = (torch.arange(R, dtype=torch.int64) % 4).cuda()
    seeds[0], draws[0] = 1234, 1
    toks = ops.sample(logits, temp, None, None, seeds, draws)
    assert toks[0].item() != 58452
    assert_plain_draws(toks, logits, temp, None, None, seeds, draws)
    top_k = torch.full((R,), -1, dtype=torch.int32).cuda()
    top_k[1::3] = 50
    top_p = torch.ones(R).cuda()
    top_p[2::3] = 0.85
    toks = ops.sample(logits, temp, top_k, top_p, seeds, draws)
    # (the kernel finds the top-p cut with weights from the hardware's 2^x: a logit right at the cut
    # may fall on either side, so the plain cut is taken a little wider)
    assert_plain_draws(toks, logits, temp, top_k, torch.clamp(top_p + 1e-4, max=1.0), seeds, draws)
    short = logits[:, :3000].contiguous()                     # one workgroup a row
    toks = ops.sample(short, temp, top_k, top_p, seeds, draws)
    assert_plain_draws(toks, short, temp, top_k, torch.clamp(top_p + 1e-4, max=1.0), seeds, draws)


@pytest.mark.parametrize("V", [50000, 50001, 152064])
def test_sampling_cuts_of_a_wide_vocabulary(V):
    """top-k and top-p over a wide row (vector loads when the row is 16-byte
    aligned, scalar ones otherwise): every drawn token lies inside the exact
    cut, and the draws reach most of what the cut keeps."""
    from servelab_amd.kernels import HipOps
    ops = HipOps(torch.float32, "cuda:0")
    R, T = 48, 0.9
    logits = 2.5 * randn(1, V, seed=V).repeat(R, 1).contiguous()
    logits[:, 1234] = logits.max() + 0.5
    temp = torch.full((R,), T).cuda()
    seeds = torch.full((R,), 99, dtype=torch.int64).cuda()
    ones, none = torch.ones(R).cuda(), torch.full((R,), -1, dtype=torch.int32).cuda()
    probs = torch.softmax(logits[0].double().cpu() / T, -1)
    sp, si = torch.sort(probs, descending=True)
    cum = torch.cumsum(sp, 0)

    def draw(top_k, top_p, rounds=20):
        got = []
        for j in range(rounds):
            draws = (torch.arange(R, dtype=torch.int64) + R * j).cuda()
            got += ops.sample(logits, temp, top_k, top_p, seeds, draws).tolist()
        return set(got)

    k = 25
    got = draw(torch.full((R,), k, dtype=torch.int32).cuda(), ones)
    assert got <= set(si[:k].tolist()) and len(got) > k // 2
    p = 0.35
    inside = set(si[(cum <= p + 1e-4) | (torch.arange(V) == 0)].tolist())
    surely = set(si[(cum <= p - 1e-4) | (torch.arange(V) == 0)].tolist())
    got = draw(none, torch.full((R,), p).cuda())
    assert got <= inside and len(got & surely) > min(len(surely), 40) // 2
    # a top_p below the largest probability keeps that entry alone
    assert draw(none, torch.full((R,), float(sp[0]) * 0.5).cuda(), rounds=2) == {1234}


@pytest.mark.parametrize("V", [8191, 8192, 12289, 40003])      # one workgroup a row below 8,192 logits, several from there
def test_sampling_rows_with_different_rules_in_one_call(V):
    """Rows of one call follow their own rule (greedy, top-k, top-p, none) when
    the cuts are searched by several workgroups a row; rows that are not
    16-byte aligned, entries at -inf and equal logits at the cut included."""
    from servelab_amd.kernels import HipOps
    ops = HipOps(torch.float32, "cuda:0")
    T = 0.8
    base = 2.0 * randn(6, V, seed=5)
    base[4, torch.randperm(V)[: V // 2].cuda()] = -math.inf
    top = base[5].max().item()
    tied = [11, 2222, V - 7]
    base[5, tied] = top + 1.0                           # three equal logits at the top
    logits = base.contiguous()
    temp = torch.tensor([0.0, T, T, T, T, T]).cuda()
    top_k = torch.tensor([-1, 1, -1, -1, 40, -1], dtype=torch.int32).cuda()
    top_p = torch.tensor([1.0, 1.0, 1e-6, 1.0, 1.0, 0.5]).cuda()
    seeds = torch.arange(6, dtype=torch.int64).cuda()
    got = [set() for _ in range(6)]
    for j in range(40):
        draws = torch.full((6,), j, dtype=torch.int64).cuda()
        toks = ops.sample(logits, temp, top_k, top_p, seeds, draws).tolist()
        assert toks == ops.sample(logits, temp, top_k, top_p, seeds, draws).tolist()
        for r, t in enumerate(toks):
            got[r].add(t)
    best = torch.argmax(logits, -1).tolist()
    assert got[0] == {best[0]} and got[1] == {best[1]} and got[2] == {best[2]}
    assert len(got[3]) > 20                               # no cut: draws spread over the row
    assert got[4] <= set(torch.topk(logits[4], 40).indices.tolist()) and len(got[4]) > 10
    probs = torch.softmax(logits[5].double().cpu() / T, -1)
    sp, si = torch.sort(probs, descending=True)
    cum = torch.cumsum(sp, 0)
    inside = set(si[(cum <= 0.5 + 1e-4) | (torch.arange(V) == 0)].tolist())
    # equal logits at the cut: the reference's sort keeps some of them, a threshold all or none
    lowest = min(logits[5, i].item() for i in inside)
    inside |= set((logits[5] >= lowest).nonzero().flatten().tolist())
    assert got[5] <= inside and set(tied) & got[5]
    # the row without a cut draws what the two-stage kernel alone draws
    draws = torch.zeros(6, dtype=torch.int64).cuda()
    assert (ops.sample(logits, temp, top_k, top_p, seeds, draws)[3]
            == ops.sample(logits, temp, None, None, seeds, draws)[3])


def test_products_of_65_to_128_rows_stay_with_the_tiled_weight():
    """Matrices of half a million elements and more take the LDS-staged kernel up to 128 rows
    (plain, gated, deferred to the norm, with rotation and cache write; float32 logits of more
    rows come from the library's float32 sums, or, without a row-major copy of the weight, in
    slices of 128 rows); smaller ones go to the library from 65 rows on."""
    from servelab_amd.kernels import HipOps
    from servelab_amd.kernels.ops import PartialSums
    ops, emu = HipOps(torch.bfloat16, "cuda:0"), EmulatedOps(torch.bfloat16)
    M, K, N = 100, 3584, 2560                        # N K = 9.2 M elements: the LDS-staged kernel's
    x = randn(M, K, dtype=torch.bfloat16, seed=1)
    w = randn(N, K, dtype=torch.bfloat16, scale=0.05, seed=2)
    weight, b = ops.prepare_weight(w), randn(N, seed=3)
    assert ops._few_rows_limit(weight) == 128
    assert ops._few_rows_limit(ops.prepare_weight(w[:256].contiguous())) == 128      # (0.9 M elements)
    assert ops._few_rows_limit(ops.prepare_weight(w[:128].contiguous())) == 64
    assert torch.equal(ops.linear(x, weight, b), ops.linear_mid(x, weight, b))
    assert rel_err(ops.linear(x, weight, b), emu.linear(x, w, b)) < 2 ** -7
    assert rel_err(ops.gated_linear(x, weight, 8), emu.silu_mul(emu.linear(x, w, None), 8)) < 2 ** -6
    delta = ops.linear(x, weight, b, defer=True)
    assert isinstance(delta, PartialSums)
    assert rel_err(ops.materialize(delta), emu.linear(x, w, b)) < 2 ** -7
    many = randn(300, K, dtype=torch.bfloat16, seed=4)
    got = ops.linear(many, weight, b, out_f32=True)
    assert got.shape == (300, N) and rel_err(got, emu.linear(many, w, b, True)) < 2e-5
    ops.weight_layout = "tiled"
    tiled_only = ops.prepare_weight(w.clone())
    assert tiled_only.w is None
    got = ops.linear(many, tiled_only, b, out_f32=True)
    assert got.shape == (300, N) and rel_err(got, emu.linear(many, w, b, True)) < 2e-5


def test_products_of_129_to_512_rows_of_matrices_of_few_rows_run_in_tiles():
    """Where the LDS-staged kernel ends, matrices of at most 8,192 rows take the kernel in tiles
    over the row-major copy, K split until every CU has a workgroup (plain, deferred as partial
    sums for the norm, q/k/v with the rotation kernel adding the sums); larger matrices, more rows,
    a model without the row-major copy and small matrices go to the library as before."""
    from servelab_amd.kernels import HipOps
    from servelab_amd.kernels.ops import PartialSums
    ops, emu = HipOps(torch.bfloat16, "cuda:0"), EmulatedOps(torch.bfloat16)
    K, N = 1024, 8192
    w = randn(N, K, dtype=torch.bfloat16, scale=0.05, seed=2)
    weight, b = ops.prepare_weight(w), randn(N, seed=3)
    for M in (129, 300, 512):
        x = randn(M, K, dtype=torch.bfloat16, seed=M)
        shares, square = ops._block_plan(M, N, K, weight)
        assert shares == max(1, min(K // 64 // 3, ops._num_cus // (N // 128 * -(-M // 256)))) and not square
        assert torch.equal(ops.linear(x, weight, b), ops.linear_block(x, weight, b, ks=shares))
        assert rel_err(ops.linear(x, weight, b), emu.linear(x, w, b)) < 2 ** -7
        delta = ops.linear(x, weight, b, defer=True)
        assert isinstance(delta, PartialSums) and delta.parts.shape == (shares, M, N)
        assert rel_err(ops.materialize(delta), emu.linear(x, w, b)) < 2 ** -7
    assert not ops._block_plan(128, N, K, weight) and not ops._block_plan(513, N, K, weight)
    assert not ops._block_plan(300, 8208, K, ops.prepare_weight(randn(8208, K, dtype=torch.bfloat16)))
    assert not ops._block_plan(300, 256, K, ops.prepare_weight(w[:256].contiguous()))
    # rows of 8,192 values and more (a down projection): tiles of 256 x 256 from 257 rows on, further up
    # than the others, as long as tiles and shares fill three quarters of the CUs
    K2, N2 = 8192, 1024
    w2 = randn(N2, K2, dtype=torch.bfloat16, scale=0.02, seed=5)
    long_rows, b2 = ops.prepare_weight(w2), randn(N2, seed=6)
    ops._num_cus = 64
    assert ops._block_plan(256, N2, K2, long_rows) == (8, False)
    assert ops._block_plan(257, N2, K2, long_rows) == (8, True) and ops._block_plan(700, N2, K2, long_rows) == (5, True)
    assert ops._block_plan(1536, N2, K2, long_rows) == (2, True) and not ops._block_plan(1537, N2, K2, long_rows)
    ops._num_cus = 256
    assert ops._block_plan(700, N2, K2, long_rows) == (16, True)
    assert ops._block_plan(700, 512, K2, ops.prepare_weight(w2[:512].contiguous())) is None    # 6 tiles x 16 shares: too few
    for M in (300, 700):
        x = randn(M, K2, dtype=torch.bfloat16, seed=M)
        shares, square = ops._block_plan(M, N2, K2, long_rows)
        assert torch.equal(ops.linear(x, long_rows, b2), ops.linear_block(x, long_rows, b2, ks=shares, square=square))
        assert rel_err(ops.linear(x, long_rows, b2), emu.linear(x, w2, b2)) < 2 ** -7
        delta = ops.linear(x, long_rows, b2, defer=True)
        assert isinstance(delta, PartialSums) and delta.parts.shape == (shares, M, N2)
        assert rel_err(ops.materialize(delta), emu.linear(x, w2, b2)) < 2 ** -7
    ops.weight_layout = "tiled"
    assert not ops._block_plan(300, N, K, ops.prepare_weight(w.clone()))
    ops.use_block_products = False
    assert not ops._block_plan(300, N, K, weight)


@pytest.mark.parametrize("M,N,K,ks", [(17, 3584, 3584, 16), (64, 3584, 18944, 12), (65, 4608, 3584, 7), (128, 520, 640, 3),
                                      (129, 136, 64, 1), (160, 4608, 3584, 1), (300, 3584, 3584, 4), (512, 1000, 640, 2),
                                      (513, 1000, 640, 3), (700, 260, 128, 1), (200, 1001, 192, 2), (256, 130, 64, 1)])
@pytest.mark.parametrize("square", [False, True])
def test_products_in_tiles_over_the_row_major_copy(M, N, K, ks, square):
    """The kernel alone in both of its tile shapes (256 x 128 with eight wavefronts and a ring of
    three stages, 256 x 256 with sixteen and a ring of two), ragged in rows and columns, with and
    without a split of K, a bias, float32 output and partial sums."""
    from servelab_amd.kernels import HipOps
    ops = HipOps(torch.bfloat16, "cuda:0")
    x = randn(M, K, dtype=torch.bfloat16, seed=1)
    w = randn(N, K, dtype=torch.bfloat16, scale=0.05, seed=2)
    b = randn(N, seed=3)
    ref = x.float() @ w.float().T
    assert rel_err(ops.linear_block(x, w, b, out_f32=True, ks=ks, square=square), ref + b) < 2e-5
    assert rel_err(ops.linear_block(x, w, None, ks=ks, square=square), ref) < 2 ** -7
    assert rel_err(ops.linear_block(x, w, b, ks=1, square=square), ref + b) < 2 ** -7
    parts = ops.linear_block(x, w, b, ks=ks, partial=True, square=square)
    assert parts.parts.shape == (ks, M, N) and parts.bias is b
    assert rel_err(parts.parts.sum(0) + b, ref + b) < 2e-5
    assert rel_err(ops.materialize(parts), ref + b) < 2 ** -7


@pytest.mark.parametrize("M,N,K", [(2, 130, 48), (8, 3584, 3584), (33, 200, 64), (64, 100, 96), (65, 100, 96),
                                   (128, 128, 16), (300, 1000, 352), (2048, 3584, 3584), (130, 70, 1024)])
def test_float32_product_on_the_matrix_cores(M, N, K):
    """Float32 products of many rows (v_mfma_f32_32x32x2_f32): against float64 as
    exact as the plain FMA kernel's float32 sums of K terms (a reduced-precision
    matrix mode would be a thousand times off); ragged edges of both tiles."""
    from servelab_amd.kernels import HipOps
    ops = HipOps(torch.float32, "cuda:0")
    x, w, b = randn(M, K, seed=1), randn(N, K, scale=0.1, seed=2), randn(N, seed=3)
    ref = (x.double() @ w.double().T + b.double())
    for bias in (None, b):
        got = ops.linear_f32_mfma(x, w, bias)
        want = ref if bias is not None else ref - b.double()
        assert got.dtype == torch.float32 and got.shape == (M, N)
        err = ((got.double() - want).abs().max() / want.abs().max()).item()
        plain = ((ops.linear_tiled(x, w, bias).double() - want).abs().max() / want.abs().max()).item()
        assert err < max(1.5 * plain, 1e-6), (err, plain)
        if M >= ops.F32_MFMA_MIN_M:
            assert torch.equal(got, ops.linear(x, w, bias))      # the float32 table's choice at these sizes


@pytest.mark.parametrize("N,K", [(200, 96), (1000, 352), (2560, 3584)])
def test_products_at_every_boundary_of_the_row_counts(N, K):
    """ops.linear / gated_linear / deferred products at each row count where the
    bfloat16 table changes kernels (few-rows, wide, LDS-staged, padded library),
    for a small, a medium and a large matrix: always the plain product."""
    from servelab_amd.kernels import HipOps
    ops, emu = HipOps(torch.bfloat16, "cuda:0"), EmulatedOps(torch.bfloat16)
    w = randn(N, K, dtype=torch.bfloat16, scale=0.05, seed=2)
    weight, b = ops.prepare_weight(w), randn(N, seed=3)
    gain = 1 + 0.1 * randn(N, seed=4)
    for M in (1, 8, 9, 16, 17, 32, 33, 64, 65, 96, 97, 128, 129, 160, 511, 512, 513):
        x = randn(M, K, dtype=torch.bfloat16, seed=M)
        ref = emu.linear(x, w, b, True)
        assert rel_err(ops.linear(x, weight, b), ref) < 2 ** -7, M
        assert rel_err(ops.linear(x, weight, b, out_f32=True), ref) < 2 ** -7, M
        assert rel_err(ops.materialize(ops.linear(x, weight, b, defer=True)), ref) < 2 ** -7, M
        if N % 16 == 0:
            assert rel_err(ops.gated_linear(x, weight, 8), emu.silu_mul(emu.linear(x, w, None), 8)) < 2 ** -6, M
        # a deferred product through the norm that adds it
        resid = randn(M, N, seed=5)
        want = resid + ref
        got = ops.add_rmsnorm(resid, ops.linear(x, weight, b, defer=True), gain, 1e-6)
        assert rel_err(resid, want) < 2 ** -7, M
        normed = want * torch.rsqrt(want.pow(2).mean(-1, keepdim=True) + 1e-6) * gain
        assert rel_err(got, normed) < 2 ** -6, M
