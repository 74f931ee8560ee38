"""Launch order of tiles (default = XCD remap + tl.swizzle2d, and the super-block order) and the persistent schedule.

CPU part: both orders are bijections for every grid (brute force through the C ABI's host copy of the device
functions), the default order equals the oracle's restatement of tl.swizzle2d behind the XCD remap, and the super-block
order has the locality it is built for.  GPU part: every schedule gives the bits the default schedule gives."""
import itertools

import pytest
import torch

import oracle
from tritonix_amd import _C
from tritonix_amd.kernel import cdiv, out_dtype_for
from tritonix_amd.ops.matmul import matmul_kernel
from tritonix_amd.ops.swiglu import glu_kernel


@pytest.mark.parametrize("schedule", [_C.SCHED_DEFAULT, _C.SCHED_SUPERBLOCK])
def test_launch_order_is_a_bijection_for_every_grid(schedule):
    grids = list(itertools.product(range(1, 21), range(1, 21))) + [(32, 32), (16, 112), (33, 17), (17, 49), (64, 5), (3, 70)]
    for tm, tn in grids:
        for gm in ((1, 4, 8) if schedule == _C.SCHED_DEFAULT and tm * tn <= 200 else (8,)):
            seen = {_C.tile_coords(schedule, i, tm, tn, gm) for i in range(tm * tn)}
            assert len(seen) == tm * tn, (tm, tn, gm)
            assert all(0 <= a < tm and 0 <= b < tn for a, b in seen)
    with pytest.raises(ValueError):
        _C.tile_coords(schedule, 12, 3, 4)          # id past the grid


def test_default_order_is_swizzle2d_behind_the_xcd_remap():
    for tm, tn, gm in [(4, 4, 2), (32, 32, 8), (16, 112, 4), (7, 9, 3), (1, 32, 8)]:
        for i in range(tm * tn):
            logical = oracle.xcd_remap(i, tm * tn)
            assert _C.tile_coords(0, i, tm, tn, gm) == oracle.swizzle2d(logical // tn, logical % tn, tm, tn, gm)


def test_superblock_order_keeps_rounds_and_xcds_local():
    """32x32 tiles (the 8192^3 problem with 256x256 tiles): a round of 256 consecutive ids is one 16x16 super-block,
    consecutive rounds share a block row or a block column, and the ids of one XCD (congruent mod 8) inside a round
    form an 8x4 sub-block, i.e. 12 operand panels through that XCD's L2."""
    rounds = []
    for r in range(4):
        tiles = [_C.tile_coords(_C.SCHED_SUPERBLOCK, r * 256 + i, 32, 32) for i in range(256)]
        rows, cols = {t[0] for t in tiles}, {t[1] for t in tiles}
        assert len(rows) == 16 and len(cols) == 16 and max(rows) - min(rows) == 15 and max(cols) - min(cols) == 15
        rounds.append((min(rows), min(cols)))
        for x in range(8):
            mine = tiles[x::8]
            assert len({t[0] for t in mine}) == 8 and len({t[1] for t in mine}) == 4
    assert rounds == [(0, 0), (0, 16), (16, 16), (16, 0)]
    for (r0, c0), (r1, c1) in zip(rounds, rounds[1:]):
        assert r0 == r1 or c0 == c1
    # the default order, for comparison, touches every block row of A in every round
    first_round = {_C.tile_coords(0, i, 32, 32)[0] for i in range(256)}
    assert len(first_round) == 32


def test_persistent_needs_a_built_variant_and_no_split():
    import ctypes

    lib = _C.load()

    def status(**kw):
        g = _C.GemmArgs()
        base = dict(m=1024, n=1024, k=1024, stride_am=1024, stride_ak=1, stride_bk=1024, stride_bn=1, stride_cm=1024,
                    stride_cn=1, in_dtype=_C.BF16, out_dtype=_C.BF16, block_m=256, block_n=128, block_k=64, group_m=8,
                    split_k=1, num_stages=2, num_warps=4, epilogue=_C.EPI_NONE, schedule=_C.SCHED_PERSISTENT)
        base.update(kw)
        for k, v in base.items():
            setattr(g, k, v)
        return lib.tnx_gemm_supported(ctypes.byref(g)), lib.tnx_gemm_lds_bytes(ctypes.byref(g))

    ring = 2 * (256 * 64 + 64 * 128) * 2
    assert status() == (_C.OK, ring + 4 * 16 * 256)                           # ring + the epilogue's own strips
    assert status(schedule=0)[1] == ring
    assert status(block_n=256)[0] == _C.E_UNSUPPORTED                     # 256x256: its accumulators leave no registers for the tile loop
    assert status(split_k=2)[0] == _C.E_UNSUPPORTED                       # persistent tiles are never cut
    assert status(k=64)[0] == _C.E_UNSUPPORTED                            # fewer K slabs than ring stages
    assert status(block_m=64, block_n=64, num_stages=4)[0] == _C.E_UNSUPPORTED   # small tiles have no persistent variant
    assert status(stride_ak=2)[0] == _C.E_UNSUPPORTED                     # DMA layout only
    assert status(schedule=8)[0] == _C.E_INVALID
    assert any("persistent" in n for n in _C.kernel_names())


# ---------------------------------------------------------------------------------------------------------------------
def cfg(bm, bn, bk, nw, st, gm=8, **extra):
    return dict(block_m=bm, block_n=bn, block_k=bk, group_m=gm, num_stages=st, num_warps=nw, **extra)


def launch(kernel, a, b, c, config, **kw):
    m, k = a.shape
    n = b.shape[1]
    grid = (cdiv(m, config["block_m"]), cdiv(n, config["block_n"]))
    kernel[grid](a, b, c, m, n, k, a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1),
                 **config, **kw)
    torch.cuda.synchronize()
    return c


def gemm(a, b, config):
    c = torch.full((a.shape[0], b.shape[1]), 7, device=a.device, dtype=out_dtype_for(a.dtype))
    return launch(matmul_kernel, a, b, c, config)


SCHEDULES = [dict(persistent=1), dict(superblock=1), dict(persistent=1, superblock=1)]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tile", [(torch.bfloat16, (128, 256, 64, 4, 2)), (torch.float16, (128, 128, 64, 4, 3)),
                                        (torch.bfloat16, (256, 128, 64, 4, 2)), (torch.int8, (256, 128, 128, 4, 2)),
                                        (torch.int8, (128, 128, 128, 4, 2))],
                         ids=lambda v: str(v).replace("torch.", ""))
@pytest.mark.parametrize("shape", [(2304, 2560, 1024), (1000, 4624, 512), (256, 256, 256), (4352, 4352, 256)],
                         ids=lambda s: "x".join(map(str, s)))
def test_every_schedule_gives_the_bits_of_the_default_schedule(device, dtype, tile, shape):
    m, n, k = shape
    g = torch.Generator("cpu").manual_seed(m + 3 * n + 7 * k)
    if dtype == torch.int8:
        a = torch.randint(-127, 128, (m, k), generator=g, dtype=torch.int8)
        b = torch.randint(-127, 128, (k, n), generator=g, dtype=torch.int8)
    else:
        a = torch.randn(m, k, generator=g).to(dtype)
        b = (torch.randn(k, n, generator=g) / k ** 0.5).to(dtype)
    ad, bd = a.to(device), b.to(device)
    want = gemm(ad, bd, cfg(*tile))
    rows = torch.arange(0, m, max(1, m // 24))
    ref = oracle.reference_matmul(a[rows], b)
    if dtype == torch.int8:
        assert torch.equal(want[rows.to(device)].cpu(), ref)
    else:
        assert oracle.within_tolerance(want[rows.to(device)], ref)[0]
    for extra in SCHEDULES:
        got = gemm(ad, bd, cfg(*tile, **extra))
        assert torch.equal(got, want), f"{extra}: result differs from the default schedule"


@pytest.mark.gpu
@pytest.mark.parametrize("activation", ["silu", "sigmoid", "identity"])
def test_persistent_glu_epilogue(device, activation):
    x, w12 = oracle.make_inputs("C4", scale_down=4)          # x[1024,1024], w12[1024,7168]: 4 x 56 tiles of 256x128
    xd, wd = x.to(device), w12.to(device)
    outs = []
    for extra in [dict()] + SCHEDULES:
        z = torch.full((x.shape[0], w12.shape[1] // 2), 7, device=device, dtype=torch.bfloat16)
        launch(glu_kernel, xd, wd, z, cfg(256, 128, 64, 4, 2, **extra), activation=activation)
        outs.append(z)
    assert oracle.within_tolerance(outs[0], oracle.reference_glu(x, w12, activation))[0]
    for z in outs[1:]:
        assert torch.equal(z, outs[0])
    # a ragged problem: rows and gated columns that end inside a tile, output with a row pitch
    xr, wr = xd[:900], wd[:, :2 * 1300].contiguous()
    base = torch.full((900, 1300), 7, device=device, dtype=torch.bfloat16)
    launch(glu_kernel, xr, wr, base, cfg(256, 128, 64, 4, 2), activation=activation)
    wide = torch.full((900, 1304 + 8), 7, device=device, dtype=torch.bfloat16)
    view = wide[:, :1300]
    launch(glu_kernel, xr, wr, view, cfg(256, 128, 64, 4, 2, persistent=1, superblock=1), activation=activation)
    assert torch.equal(view, base) and float(wide[:, 1300:].float().min()) == 7.0


@pytest.mark.gpu
def test_schedules_at_the_benchmark_size(device):
    a, b = oracle.make_inputs("C5")
    ad, bd = a.to(device), b.to(device)
    want = gemm(ad, bd, cfg(256, 256, 128, 4, 2))
    assert torch.equal(gemm(ad, bd, cfg(256, 256, 128, 4, 2, superblock=1)), want)
    for extra in SCHEDULES:
        assert torch.equal(gemm(ad, bd, cfg(256, 128, 128, 4, 2, **extra)), want)      # integer sums: any tile, same bits


@pytest.mark.gpu
def test_atomic_reduction_of_split_k_slices(device):
    """TNX_SCHED_ATOMIC_REDUCE: the slices meet in one fp32 / int32 copy through atomic adds.  Integer results stay
    exact; float results stay inside the parity bar (only the order of the fp32 additions is free); the sum region of
    the workspace is zero again after every launch, so back-to-back launches on one workspace stay correct."""
    from tritonix_amd.ops.matmul import gemm_splitk_kernel

    a, b = oracle.make_inputs("C3")
    ad, bd = a.to(device), b.to(device)
    ref = oracle.reference_matmul(a, b)
    for split_k in (4, 8):
        for _ in range(3):
            c = torch.full((16, 4096), 7, device=device, dtype=torch.bfloat16)
            launch(gemm_splitk_kernel, ad, bd, c, cfg(64, 128, 64, 8, 3, split_k=split_k, atomic_reduce=1))
            ok, _, rel = oracle.within_tolerance(c, ref)
            assert ok and rel <= 1e-2
    a8, b8 = oracle.make_inputs("C5", scale_down=8)
    a8d, b8d = a8.to(device), b8.to(device)
    want = oracle.reference_matmul(a8, b8)
    for extra in (dict(split_k=4, tail_tiles=16), dict(split_k=2), dict(split_k=8, tail_tiles=3)):
        c = torch.full((1024, 1024), 7, device=device, dtype=torch.int32)
        launch(matmul_kernel, a8d, b8d, c, cfg(128, 128, 128, 4, 2, atomic_reduce=1, **extra))
        assert torch.equal(c.cpu(), want), extra
    # ragged rows: lanes past the last row neither add nor clear
    g = torch.Generator("cpu").manual_seed(5)
    ar = torch.randn(100, 2048, generator=g).bfloat16()
    br = (torch.randn(2048, 264, generator=g) / 45).bfloat16()
    for _ in range(2):
        c = torch.full((100, 264), 7, device=device, dtype=torch.bfloat16)
        launch(matmul_kernel, ar.to(device), br.to(device), c, cfg(128, 128, 64, 4, 2, split_k=3, atomic_reduce=1))
        assert oracle.within_tolerance(c, oracle.reference_matmul(ar, br))[0]


# ---------------------------------------------------------------------------------------------------------------------
# the 192x192, 192x256 and 256x192 tiles: rows of 24 chunks in the B slab, 6 MFMA tiles across a wave -- the tiles whose
# sides are not powers of two
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=lambda v: str(v).replace("torch.", ""))
@pytest.mark.parametrize("bm,bn,waves,stages", [(192, 192, 4, 2), (192, 192, 4, 3), (192, 192, 8, 2), (192, 192, 8, 3),
                                                (192, 256, 4, 2), (192, 256, 8, 2), (256, 192, 4, 2), (256, 192, 8, 2)])
def test_the_192_tiles_give_the_bits_of_the_128_tile(device, dtype, bm, bn, waves, stages):
    """Every tile with a 64-deep K slab adds the same products in the same order, so the results must agree bit for bit:
    whole and ragged problems, the super-block order, K cut for all tiles and for the last ones only, k-contiguous B,
    the gated epilogue."""
    from tritonix_amd.ops.matmul import gemm_splitk_kernel

    for (m, n, k) in [(384, 576, 256), (1000, 1100, 520), (3072, 3072, 512), (190, 194, 64), (2880, 200, 1024)]:
        g = torch.Generator("cpu").manual_seed(m + n + k)
        a = torch.randn(m, k, generator=g).to(dtype)
        b = (torch.randn(k, n, generator=g) / k ** 0.5).to(dtype)
        ad, bd = a.to(device), b.to(device)
        want = gemm(ad, bd, cfg(128, 128, 64, 4, 2))
        rows = torch.arange(0, m, max(1, m // 16))
        assert oracle.within_tolerance(want[rows.to(device)], oracle.reference_matmul(a[rows], b))[0]
        tile = (bm, bn, 64, waves, stages)
        assert torch.equal(gemm(ad, bd, cfg(*tile)), want), (m, n, k, "plain")
        assert torch.equal(gemm(ad, bd, cfg(*tile, superblock=1)), want), (m, n, k, "super-block order")
        wt = bd.t().contiguous()                                   # B as the transposed view of an [n, k] weight
        assert torch.equal(gemm(ad, wt.t(), cfg(*tile)), want), (m, n, k, "k-contiguous B")
        if k >= 512:
            # K cut: fp32 partial sums are added in slice order, not in one chain; compare with the same cut on the 128 tile
            tiles = cdiv(m, bm) * cdiv(n, bn)
            for extra in (dict(split_k=2), dict(split_k=4, tail_tiles=min(3, tiles))):
                c = torch.full((m, n), 7, device=device, dtype=dtype)
                launch(gemm_splitk_kernel, ad, bd, c, cfg(*tile, **extra))
                assert oracle.within_tolerance(c[rows.to(device)], oracle.reference_matmul(a[rows], b))[0], (m, n, k, extra)
        if n % 2 == 0:
            z = torch.full((m, n // 2), 7, device=device, dtype=dtype)
            z128 = torch.full((m, n // 2), 7, device=device, dtype=dtype)
            launch(glu_kernel, ad, bd, z, cfg(*tile), activation="silu")
            launch(glu_kernel, ad, bd, z128, cfg(128, 128, 64, 4, 2), activation="silu")
            assert torch.equal(z, z128), (m, n, k, "gated")


@pytest.mark.gpu
@pytest.mark.parametrize("bm,bn,stages", [(192, 256, 2), (256, 192, 2), (192, 192, 2), (192, 192, 3)])
@pytest.mark.parametrize("waves", [4, 8])
def test_the_int8_192_tiles_are_exact(device, waves, bm, bn, stages):
    for (m, n, k) in [(384, 512, 256), (1000, 1100, 520), (3072, 1024, 1024), (190, 200, 128)]:
        g = torch.Generator("cpu").manual_seed(m + n + k)
        a = torch.randint(-127, 128, (m, k), generator=g, dtype=torch.int8)
        b = torch.randint(-127, 128, (k, n), generator=g, dtype=torch.int8)
        ad, bd = a.to(device), b.to(device)
        want = gemm(ad, bd, cfg(128, 128, 128, 4, 2))
        rows = torch.arange(0, m, max(1, m // 16))
        assert torch.equal(want[rows.to(device)].cpu(), oracle.reference_matmul(a[rows], b))
        assert torch.equal(gemm(ad, bd, cfg(bm, bn, 128, waves, stages)), want), (m, n, k)
        assert torch.equal(gemm(ad, bd, cfg(bm, bn, 128, waves, stages, superblock=1)), want), (m, n, k, "super-block order")
