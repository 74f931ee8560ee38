"""GPU parity: the HIP kernels, called through the C ABI (HipKernel -> tnx_gemm), against the CPU oracle on
the same seeded inputs.  Integer work must be bit-exact; floating point must satisfy
|out - ref| <= 1e-2*|ref| + 1e-2*rms(ref) and max|out-ref|/max|ref| <= 1e-2 against the fp32 CPU matmul."""
import pytest
import torch

import oracle
from tritonix_amd.kernel import cdiv, out_dtype_for
from tritonix_amd.ops.matmul import gemm_splitk_kernel, matmul_kernel
from tritonix_amd.ops.swiglu import glu_kernel
from tritonix_amd.testing import OutOfResources

pytestmark = pytest.mark.gpu

REL = 1e-2


def cfg(bm, bn, bk, nw, st, gm=8, **extra):
    return dict(block_m=bm, block_n=bn, block_k=bk, group_m=gm, num_stages=st, num_warps=nw, **extra)


def run(kernel, a, b, c, config, **kw):
    m, k = a.shape
    n = b.shape[1]
    grid = (cdiv(m, config["block_m"]), cdiv(n, config["block_n"]))
    kernel[grid](a, b, c, m, n, k, a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1),
                 **config, **kw)
    torch.cuda.synchronize()
    return c


def gemm(a, b, config, kernel=matmul_kernel):
    c = torch.full((a.shape[0], b.shape[1]), 7, device=a.device, dtype=out_dtype_for(a.dtype))
    return run(kernel, a, b, c, config)


def check_fp(out, ref):
    ok, maxerr, rel = oracle.within_tolerance(out, ref, REL)
    assert ok, f"outside tolerance: max err {maxerr}, max err / max|ref| {rel}"
    assert rel <= REL


def whole_matrix_identity(out, a64, b64, rel_bound=2e-3):
    """A check that touches every element of a result too large for an element-wise CPU comparison:
    row sums  C.1 == A.(B.1)  and column sums  1.C == (1.A).B , right-hand sides in float64 on the CPU.
    The left-hand sides differ from them only by the 16-bit rounding of each output element, whose sum over a
    row has a standard deviation of about 2^-9 * rms(C) * sqrt(n): the bound is set at many times that,
    while a tile left unwritten or written to the wrong place moves a sum by the size of the tile's content."""
    c = out.double().cpu()
    n_cols = c.shape[1]
    want_rows = a64 @ b64.sum(dim=1)
    want_cols = a64.sum(dim=0) @ b64
    scale = float(c.abs().mean()) * n_cols ** 0.5          # size of a row sum of independent entries
    assert float((c.sum(dim=1) - want_rows).abs().max()) <= rel_bound * scale * 8
    scale_c = float(c.abs().mean()) * c.shape[0] ** 0.5
    assert float((c.sum(dim=0) - want_cols).abs().max()) <= rel_bound * scale_c * 8


F16_TILES = [cfg(128, 128, 64, 4, 2), cfg(128, 128, 64, 4, 3), cfg(256, 256, 64, 4, 2), cfg(64, 128, 64, 4, 3, gm=4),
             cfg(128, 128, 64, 8, 2), cfg(256, 256, 64, 8, 2), cfg(64, 128, 64, 8, 3)]


# ---- C1: fp16 1024x512 @ 512x768, full size ------------------------------------------
@pytest.mark.parametrize("config", F16_TILES, ids=lambda c: "x".join(str(v) for v in c.values()))
def test_c1_fp16_full_size(device, config):
    a, b = oracle.make_inputs("C1")
    out = gemm(a.to(device), b.to(device), config)
    assert out.dtype == torch.float16
    check_fp(out, oracle.reference_matmul(a, b))


# ---- C2: bf16 square ------------------------------------------------------------------
@pytest.mark.parametrize("config", [cfg(256, 256, 64, 4, 2), cfg(256, 256, 64, 8, 2), cfg(128, 128, 64, 4, 3)],
                         ids=lambda c: "x".join(str(v) for v in c.values()))
def test_c2_bf16_square_1024(device, config):
    a, b = oracle.make_inputs("C2", scale_down=8)
    check_fp(gemm(a.to(device), b.to(device), config), oracle.reference_matmul(a, b))


def test_c2_bf16_full_size_rows_and_linearity(device):
    a, b = oracle.make_inputs("C2")
    ad, bd = a.to(device), b.to(device)
    config = cfg(256, 256, 64, 4, 2)
    out = gemm(ad, bd, config)
    # one row out of every 256-row tile (at a different offset inside each) plus the edges of the matrix
    rows = torch.tensor(sorted({0, 1, 255, 256, 4095, 4096, 8190, 8191} | {256 * t + (37 * t + 5) % 256 for t in range(32)}))
    check_fp(out[rows.to(device)], oracle.reference_matmul(a[rows], b))
    whole_matrix_identity(out, a.double(), b.double())
    # scaling an operand by a power of two scales every product and partial sum exactly
    out2 = gemm(ad * 2, bd, config)
    assert torch.equal(out2, out * 2)
    # and a second launch reproduces the first bit for bit
    assert torch.equal(gemm(ad, bd, config), out)


# ---- C3: skinny split-K ---------------------------------------------------------------
@pytest.mark.parametrize("split_k", [2, 4, 8, 16])
def test_c3_splitk_full_size(device, split_k):
    a, b = oracle.make_inputs("C3")
    ad, bd = a.to(device), b.to(device)
    config = cfg(64, 128, 64, 4, 3, split_k=split_k)
    out = gemm(ad, bd, config, kernel=gemm_splitk_kernel)
    assert out.shape == (16, 4096) and out.dtype == torch.bfloat16
    check_fp(out, oracle.reference_matmul(a, b))
    # workspace partials summed in a fixed order: run-to-run identical, no atomics
    assert torch.equal(gemm(ad, bd, config, kernel=gemm_splitk_kernel), out)


def test_splitk_matches_non_split_within_rounding(device):
    a, b = oracle.make_inputs("C3", scale_down=4)
    ad, bd = a.to(device), b.to(device)
    plain = gemm(ad, bd, cfg(64, 128, 64, 4, 3))
    split = gemm(ad, bd, cfg(64, 128, 64, 4, 3, split_k=7), kernel=gemm_splitk_kernel)   # 56 slabs / 7
    ref = oracle.reference_matmul(a, b)
    check_fp(split, ref)
    check_fp(plain, ref)
    # more splits than K slabs: the empty splits must contribute zeros
    tiny_a, tiny_b = ad[:, :128].contiguous(), bd[:128].contiguous()
    check_fp(gemm(tiny_a, tiny_b, cfg(64, 128, 64, 4, 3, split_k=16), kernel=gemm_splitk_kernel),
             oracle.reference_matmul(tiny_a, tiny_b))


# ---- C4: fused GLU --------------------------------------------------------------------
@pytest.mark.parametrize("activation", ["silu", "sigmoid", "identity"])
@pytest.mark.parametrize("config", [cfg(256, 256, 64, 4, 2), cfg(128, 128, 64, 4, 3), cfg(128, 128, 64, 8, 2)],
                         ids=lambda c: "x".join(str(v) for v in c.values()))
def test_c4_glu_scaled(device, activation, config):
    x, w12 = oracle.make_inputs("C4", scale_down=8)     # x[512,512], w12[512,3584]
    z = torch.full((x.shape[0], w12.shape[1] // 2), 7, device=device, dtype=torch.bfloat16)
    run(glu_kernel, x.to(device), w12.to(device), z, config, activation=activation)
    check_fp(z, oracle.reference_glu(x, w12, activation))


@pytest.mark.parametrize("activation", ["silu", "sigmoid"])
@pytest.mark.parametrize("config", [cfg(256, 256, 64, 8, 2), cfg(128, 128, 64, 4, 3)],
                         ids=lambda c: "x".join(str(v) for v in c.values()))
def test_glu_ragged_operands_on_the_dma_path(device, activation, config):
    """K no multiple of block_k, rows of x and of the interleaved weight off 16 bytes, a gated width that ends inside a
    chunk: the last K slab is loaded chunk by chunk.  Same bits as the launch on zero-padded, aligned copies."""
    g = torch.Generator("cpu").manual_seed(77)
    m, k, n2 = 700, 1030, 2 * 1301
    x = torch.randn(m, k, generator=g).bfloat16()
    w12 = (0.05 * torch.randn(k, n2, generator=g)).bfloat16()
    z = torch.full((m, n2 // 2), 7, device=device, dtype=torch.bfloat16)
    run(glu_kernel, x.to(device), w12.to(device), z, config, activation=activation)
    check_fp(z, oracle.reference_glu(x, w12, activation))
    kp, np2 = 1088, 2 * 1304
    xp = torch.zeros((m, kp), dtype=torch.bfloat16)
    wp = torch.zeros((kp, np2), dtype=torch.bfloat16)
    xp[:, :k] = x
    wp[:k, :n2] = w12
    zp = torch.full((m, np2 // 2), 7, device=device, dtype=torch.bfloat16)
    run(glu_kernel, xp.to(device), wp.to(device), zp, config, activation=activation)
    assert torch.equal(z, zp[:, :n2 // 2])


def test_c4_glu_full_size_rows(device):
    x, w12 = oracle.make_inputs("C4")
    xd, wd = x.to(device), w12.to(device)
    rows = torch.tensor(sorted({0, 255, 256, 2047, 2048, 4095} | {256 * t + (53 * t + 11) % 256 for t in range(16)}))
    for act in ("silu", "sigmoid"):
        z = torch.empty((4096, 14336), device=device, dtype=torch.bfloat16)
        run(glu_kernel, xd, wd, z, cfg(256, 256, 64, 4, 2), activation=act)
        check_fp(z[rows.to(device)], oracle.reference_glu(x[rows], w12, act))
    # every element of a whole result: the un-activated gate makes Z = (x W1) * (x W2) elementwise, and the plain
    # GEMM of the same operands through the same tile gives both factors; the products must agree within the two
    # roundings, everywhere (the plain kernel is itself checked over the whole matrix by the test below)
    z = torch.empty((4096, 14336), device=device, dtype=torch.bfloat16)
    run(glu_kernel, xd, wd, z, cfg(256, 256, 64, 4, 2), activation="identity")
    y = gemm(xd, wd, cfg(256, 256, 64, 4, 2))
    prod = y[:, 0::2].float() * y[:, 1::2].float()
    err = (z.float() - prod).abs()
    assert bool((err <= 2e-2 * prod.abs() + 1e-2 * prod.pow(2).mean().sqrt()).all())
    whole_matrix_identity(y, x.double(), w12.double())


# ---- C5: int8 -> int32, bit-exact -----------------------------------------------------
@pytest.mark.parametrize("config", [cfg(256, 256, 128, 4, 2), cfg(128, 128, 128, 4, 2), cfg(256, 256, 128, 8, 2),
                                    cfg(64, 128, 128, 4, 3)], ids=lambda c: "x".join(str(v) for v in c.values()))
def test_c5_int8_exact_1024(device, config):
    a, b = oracle.make_inputs("C5", scale_down=8)
    out = gemm(a.to(device), b.to(device), config)
    assert out.dtype == torch.int32
    assert torch.equal(out.cpu(), oracle.reference_matmul(a, b))


def test_c5_int8_full_size_rows_exact(device):
    a, b = oracle.make_inputs("C5")
    out = gemm(a.to(device), b.to(device), cfg(256, 256, 128, 4, 2))
    rows = torch.tensor([0, 255, 256, 4095, 4096, 8191] + list(range(77, 8000, 997)))
    assert torch.equal(out[rows.to(device)].cpu(), oracle.reference_matmul(a[rows], b))
    # a checksum over the whole result: sum_j C[i,j] == A[i,:] . (B @ 1)
    colsum = b.double().sum(dim=1)
    assert torch.equal(out.sum(dim=1, dtype=torch.int64).cpu(), (a.double() @ colsum).to(torch.int64))


def test_int8_extremes(device):
    a = torch.full((64, 8192), -127, dtype=torch.int8)
    b = torch.full((8192, 128), -127, dtype=torch.int8)
    out = gemm(a.to(device), b.to(device), cfg(64, 128, 128, 4, 3))
    assert int(out.min()) == int(out.max()) == 8192 * 127 * 127


# ---- edges: ragged shapes, strides, tiny and empty problems ----------------------------
GENERIC = cfg(128, 128, 64, 4, 2)       # built with the element-wise loader as well


@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (1, 8, 64), (16, 24, 40), (100, 264, 200), (129, 257, 65),
                                   (300, 264, 192), (37, 1000, 333)])
def test_ragged_shapes_bf16(device, m, n, k):
    g = torch.Generator("cpu").manual_seed(m * 131 + n * 17 + k)
    a = torch.randn(m, k, generator=g).bfloat16()
    b = torch.randn(k, n, generator=g).bfloat16()
    check_fp(gemm(a.to(device), b.to(device), GENERIC), oracle.reference_matmul(a, b))


@pytest.mark.parametrize("m,n,k", [(5, 7, 3), (33, 17, 100)])
def test_tiny_shapes_against_the_tile_walking_oracle(device, m, n, k):
    g = torch.Generator("cpu").manual_seed(9)
    a = torch.randn(m, k, generator=g).half()
    b = torch.randn(k, n, generator=g).half()
    walk = torch.from_numpy(oracle.tiled_matmul(a.float().numpy(), b.float().numpy(), 32, 32, 16, 4))
    check_fp(gemm(a.to(device), b.to(device), GENERIC), walk)
    ai = torch.randint(-127, 128, (m, k), generator=g, dtype=torch.int8)
    bi = torch.randint(-127, 128, (k, n), generator=g, dtype=torch.int8)
    got = gemm(ai.to(device), bi.to(device), cfg(128, 128, 128, 4, 2))
    assert torch.equal(got.cpu(), torch.from_numpy(oracle.tiled_matmul_i8(ai.numpy(), bi.numpy())))


def test_strided_operands_and_output(device):
    g = torch.Generator("cpu").manual_seed(11)
    at = torch.randn(192, 160, generator=g).bfloat16()       # use a = at.T (column-major A)
    bt = torch.randn(136, 192, generator=g).bfloat16()       # use b = bt.T (column-major B)
    a, b = at.t(), bt.t()
    ref = oracle.reference_matmul(a, b)
    check_fp(gemm(a.to(device).t().contiguous().t(), b.to(device), GENERIC), ref)   # contiguous a, strided b
    ad, bd = at.to(device).t(), bt.to(device).t()
    assert ad.stride() == (1, 160) and bd.stride() == (1, 192)
    check_fp(gemm(ad, bd, GENERIC), ref)
    # output with a row pitch and a column step
    buf = torch.zeros(160, 2 * 136 + 6, device=device, dtype=torch.bfloat16)
    c = buf[:, 3:3 + 2 * 136:2]
    run(matmul_kernel, ad, bd, c, GENERIC)
    check_fp(c, ref)
    assert float(buf[:, :3].abs().sum()) == 0 and float(buf[:, 4::2].abs().sum()) == 0
    # row-major operands whose rows are padded stay on the fast loader
    wide_a = torch.zeros(256, 512 + 64, device=device, dtype=torch.bfloat16)
    wide_b = torch.zeros(512, 384 + 8, device=device, dtype=torch.bfloat16)
    a2 = torch.randn(256, 512, generator=g).bfloat16()
    b2 = torch.randn(512, 384, generator=g).bfloat16()
    wide_a[:, :512] = a2.to(device)
    wide_b[:, :384] = b2.to(device)
    check_fp(gemm(wide_a[:, :512], wide_b[:, :384], cfg(128, 128, 64, 4, 3)), oracle.reference_matmul(a2, b2))


def test_empty_problems(device):
    a = torch.zeros(0, 64, device=device, dtype=torch.bfloat16)
    b = torch.zeros(64, 32, device=device, dtype=torch.bfloat16)
    assert gemm(a, b, GENERIC).shape == (0, 32)
    # k == 0: the product is all zeros
    a = torch.zeros(8, 0, device=device, dtype=torch.bfloat16)
    b = torch.zeros(0, 16, device=device, dtype=torch.bfloat16)
    assert float(gemm(a, b, GENERIC).abs().sum()) == 0


def test_error_mapping_on_launch(device):
    a = torch.zeros(256, 256, device=device, dtype=torch.bfloat16)
    with pytest.raises(OutOfResources):
        gemm(a, a, cfg(256, 256, 64, 4, 3))           # 196608 B of LDS: rejected before any launch
    with pytest.raises(ValueError):
        gemm(a, a, cfg(96, 128, 64, 4, 2))            # no such tile
    with pytest.raises(ValueError):
        gemm(a[:, :200].t(), a[:200], cfg(128, 128, 64, 4, 3))   # strided A on a DMA-only tile
    with pytest.raises(ValueError):
        gemm(a.double(), a.double(), GENERIC)         # no float64 path (float32 runs as a bf16 split)
    with pytest.raises(ValueError):
        gemm(a.float(), a.float(), cfg(256, 256, 64, 4, 2))      # float32: tiles up to 128x128 only
    with pytest.raises(ValueError):
        gemm(a.cpu(), a.cpu(), GENERIC)


# ---- row-major operands the DMA loader takes with an element-wise last K slab ---------------
@pytest.mark.parametrize("dtype,tile,shape,off,pad,split", [
    (torch.bfloat16, (256, 256, 64, 4, 2), (1000, 1100, 1032), (0, 0), (0, 0), 1),      # K = 16 slabs + 8
    (torch.bfloat16, (256, 256, 64, 8, 2), (520, 1304, 1028), (0, 0), (0, 0), 1),       # rows of A 8 bytes off
    (torch.bfloat16, (256, 128, 64, 4, 3), (512, 1030, 1024), (0, 0), (0, 0), 1),       # N ends inside a chunk, K whole
    (torch.bfloat16, (128, 128, 64, 4, 3), (700, 517, 1031), (5, 7), (3, 5), 1),        # everything odd, views into larger buffers
    (torch.float16, (64, 64, 64, 4, 4), (300, 200, 40), (1, 1), (0, 0), 1),             # K shorter than one slab
    (torch.bfloat16, (128, 128, 64, 4, 3), (512, 1024, 4135), (0, 0), (0, 0), 8),       # K cut eight ways, the tail in the last slice
    (torch.bfloat16, (64, 128, 64, 8, 3), (16, 4096, 14340), (0, 0), (0, 0), 8),        # the skinny benchmark shape plus four
    (torch.int8, (256, 256, 128, 4, 2), (600, 1000, 1168), (0, 0), (0, 8), 1),          # int8: ragged K and N
    (torch.int8, (64, 128, 128, 4, 3), (64, 2051, 2064), (0, 0), (0, 13), 1),
    (torch.int8, (256, 256, 128, 4, 2), (600, 1003, 1165), (3, 5), (1, 2), 1),          # int8 rows at odd byte addresses
], ids=lambda v: str(v).replace("torch.", "").replace(" ", ""))
def test_ragged_row_major_operands_on_the_dma_path(device, dtype, tile, shape, off, pad, split):
    """What surrounds the operands in memory is NaN (int8: 77): nothing of it may reach C.  A second launch on
    zero-padded, aligned copies runs the ordinary DMA path; slab by slab both add the same products in the same
    order, so the two results have to agree bit for bit."""
    m, n, k = shape
    g = torch.Generator("cpu").manual_seed(m + 3 * n + 7 * k)
    fill = 77 if dtype == torch.int8 else float("nan")
    if dtype == torch.int8:
        a = torch.randint(-127, 128, (m, k), generator=g, dtype=dtype)
        b = torch.randint(-127, 128, (k, n), generator=g, dtype=dtype)
    else:
        a = torch.randn(m, k, generator=g).to(dtype)
        b = (torch.randn(k, n, generator=g) / k ** 0.5).to(dtype)
    abuf = torch.full((m * (k + pad[0]) + 64,), fill, dtype=dtype)
    bbuf = torch.full((k * (n + pad[1]) + 64,), fill, dtype=dtype)
    av = abuf[off[0]:off[0] + m * (k + pad[0])].view(m, k + pad[0])
    bv = bbuf[off[1]:off[1] + k * (n + pad[1])].view(k, n + pad[1])
    av[:, :k] = a
    bv[:, :n] = b
    ad = abuf.to(device)[off[0]:off[0] + m * (k + pad[0])].view(m, k + pad[0])[:, :k]
    bd = bbuf.to(device)[off[1]:off[1] + k * (n + pad[1])].view(k, n + pad[1])[:, :n]
    extra = dict(split_k=split) if split > 1 else {}
    kernel = gemm_splitk_kernel if split > 1 else matmul_kernel
    out = gemm(ad, bd, cfg(*tile, **extra), kernel=kernel)
    ref = oracle.reference_matmul(a, b)
    if dtype == torch.int8:
        assert torch.equal(out.cpu(), ref)
    else:
        assert bool(torch.isfinite(out.float()).all())
        check_fp(out, ref)
    bk = tile[2]
    kp, npad = -(-k // bk) * bk, -(-n // 16) * 16
    ap = torch.zeros((m, kp), dtype=dtype)
    bp = torch.zeros((kp, npad), dtype=dtype)
    ap[:, :k] = a
    bp[:k, :n] = b
    want = gemm(ap.to(device), bp.to(device), cfg(*tile, **extra), kernel=kernel)[:, :n]
    assert torch.equal(out, want)


# ---- K cut only for the trailing tiles (fills the last, partial wave of workgroups) ------
@pytest.mark.parametrize("tail,split_k", [(1, 2), (5, 4), (16, 4), (47, 8), (48, 2), (200, 4)])
def test_tail_tiles_split_bf16(device, tail, split_k):
    g = torch.Generator("cpu").manual_seed(tail * 100 + split_k)
    a = (torch.randn(700, 2048, generator=g) / 45.0).to(torch.bfloat16)      # 6 x 8 = 48 tiles of 128x128, ragged M
    b = torch.randn(2048, 1000, generator=g).to(torch.bfloat16)
    ref = oracle.reference_matmul(a, b)
    ad, bd = a.to(device), b.to(device)
    config = cfg(128, 128, 64, 4, 3, split_k=split_k, tail_tiles=tail)
    out = gemm(ad, bd, config, kernel=gemm_splitk_kernel)
    check_fp(out, ref)
    assert torch.equal(gemm(ad, bd, config, kernel=gemm_splitk_kernel), out)          # slices are added in slice order
    # whole tiles of the same launch are bit-identical to the plain kernel's
    plain = gemm(ad, bd, cfg(128, 128, 64, 4, 3))
    assert (out == plain).float().mean() > (48 - min(tail, 48)) / 48 - 1e-6
    # matmul_kernel takes the same two keywords
    assert torch.equal(gemm(ad, bd, config, kernel=matmul_kernel), out)


def test_tail_tiles_int8_exact_and_glu(device):
    g = torch.Generator("cpu").manual_seed(77)
    a = torch.randint(-127, 128, (520, 1024), generator=g, dtype=torch.int8)
    b = torch.randint(-127, 128, (1024, 768), generator=g, dtype=torch.int8)
    out = gemm(a.to(device), b.to(device), cfg(128, 128, 128, 4, 2, split_k=4, tail_tiles=7), kernel=gemm_splitk_kernel)
    assert torch.equal(out.cpu(), oracle.reference_matmul(a, b))
    out = gemm(a.to(device), b.to(device), cfg(256, 256, 128, 4, 2, split_k=3), kernel=gemm_splitk_kernel)
    assert torch.equal(out.cpu(), oracle.reference_matmul(a, b))
    # gated epilogue on a launch whose last tiles are cut
    x = (torch.randn(300, 1024, generator=g)).to(torch.bfloat16)
    w = (0.05 * torch.randn(1024, 1536, generator=g)).to(torch.bfloat16)
    xd, wd = x.to(device), w.to(device)
    for act in ("silu", "sigmoid"):
        z = torch.full((300, 768), 7, device=device, dtype=torch.bfloat16)
        run(glu_kernel, xd, wd, z, cfg(128, 128, 64, 4, 2), use_tf32=True, activation=act, split_k=4, tail_tiles=11)
        check_fp(z, oracle.reference_glu(x, w, act))


# ---- wavefront-level split-K kernel (m <= 16, eight K slices meet in LDS) ---------------
@pytest.mark.parametrize("m,n,k,stages,dtype", [(16, 4096, 14336, 6, torch.bfloat16), (16, 512, 2048, 3, torch.bfloat16),
                                                (5, 96, 512, 4, torch.bfloat16), (1, 32, 256, 5, torch.float16)])
def test_skinny_wave_split_kernel(device, m, n, k, stages, dtype):
    if (m, n, k) == (16, 4096, 14336):
        a, b = oracle.make_inputs("C3")
    else:
        g = torch.Generator("cpu").manual_seed(m * 7 + n)
        a = torch.randn(m, k, generator=g).to(dtype)
        b = (0.05 * torch.randn(k, n, generator=g)).to(dtype)
    config = dict(block_m=16, block_n=32, block_k=32, group_m=8, split_k=8, num_stages=stages, num_warps=8)
    out = gemm(a.to(device), b.to(device), config, kernel=gemm_splitk_kernel)
    check_fp(out, oracle.reference_matmul(a, b))
    assert torch.equal(gemm(a.to(device), b.to(device), config, kernel=gemm_splitk_kernel), out)
    with pytest.raises(ValueError):      # this kernel is the eight-way split: nothing else is accepted
        gemm(a.to(device), b.to(device), dict(config, split_k=4), kernel=gemm_splitk_kernel)
    if m < 17:
        with pytest.raises(ValueError):  # and it only takes up to sixteen rows
            big = torch.zeros(17, k, dtype=dtype, device=device)
            gemm(big, b.to(device), config, kernel=gemm_splitk_kernel)


# ---- k-contiguous B: the layout of x @ w.t() with a row-major weight ---------------------------
@pytest.mark.parametrize("dtype,tile,shape", [
    (torch.bfloat16, (256, 256, 64, 4, 2), (1024, 1024, 512)),
    (torch.bfloat16, (256, 256, 64, 4, 2), (1000, 1303, 512)),     # ragged rows and an odd number of columns
    (torch.bfloat16, (128, 128, 64, 4, 3), (300, 264, 192)),
    (torch.float16, (64, 64, 64, 4, 4), (1024, 768, 512)),
    (torch.int8, (256, 256, 128, 4, 2), (1024, 1000, 1024)),
    (torch.int8, (64, 128, 128, 4, 3), (64, 2051, 2048)),
    (torch.bfloat16, (64, 128, 64, 8, 3), (16, 4096, 14336)),      # the skinny benchmark shape against w.t(), K cut 8 ways
    (torch.bfloat16, (256, 256, 64, 4, 2), (1000, 1100, 1032)),    # K = 16 slabs + 8: the last slab is loaded chunk by chunk
    (torch.bfloat16, (128, 128, 64, 4, 3), (520, 1304, 1031)),     # rows of A and of w two bytes off 16
    (torch.int8, (256, 256, 128, 4, 2), (600, 1000, 1168)),        # int8: ragged K, rows 16-byte aligned
    (torch.bfloat16, (64, 128, 64, 8, 3), (16, 4096, 14340)),      # skinny, K cut 8 ways, ragged K
], ids=lambda v: str(v).replace("torch.", "").replace(" ", ""))
def test_k_contiguous_b_takes_its_own_dma_loader(device, dtype, tile, shape):
    m, n, k = shape
    g = torch.Generator("cpu").manual_seed(m + n + k)
    if dtype == torch.int8:
        a = torch.randint(-127, 128, (m, k), generator=g, dtype=dtype)
        w = torch.randint(-127, 128, (n, k), generator=g, dtype=dtype)
    else:
        a = torch.randn(m, k, generator=g).to(dtype)
        w = (torch.randn(n, k, generator=g) / k ** 0.5).to(dtype)
    ad, wd = a.to(device), w.to(device)
    b = wd.t()
    assert b.stride() == (1, k)
    extra = dict(split_k=8) if m == 16 else {}
    kernel = gemm_splitk_kernel if extra else matmul_kernel
    out = gemm(ad, b, cfg(*tile, **extra), kernel=kernel)
    ref = oracle.reference_matmul(a, w.t())
    if dtype == torch.int8:
        assert torch.equal(out.cpu(), ref)
    else:
        check_fp(out, ref)
    # the same products in the same order as with a row-major copy of B
    assert torch.equal(out, gemm(ad, b.contiguous(), cfg(*tile, **extra), kernel=kernel))


# ---- operands beyond 4 GiB and 2^31 elements: every byte offset is 64-bit -----------------------
@pytest.mark.parametrize("shape", [(49152, 49152, 49152), (50000, 49160, 49200)], ids=lambda s: "x".join(map(str, s)))
def test_operands_beyond_four_gibibytes(device, shape):
    """A, B and C of 4.8 GB each (the second case ragged, rows off 16 bytes).  No CPU product of that size: row sums
    C.1 == A.(B.1) and column sums 1.C == (1.A).B in float64 on the GPU (chunked reductions), and the far corner of
    C element by element.  The bounds are those of whole_matrix_identity: many times the 16-bit output rounding,
    far below what a tile written to the wrong place would move."""
    m, n, k = shape
    torch.manual_seed(0)
    a = torch.empty((m, k), device=device, dtype=torch.bfloat16)
    b = torch.empty((k, n), device=device, dtype=torch.bfloat16)
    for i in range(0, m, 4096):
        a[i:i + 4096] = (torch.randn(min(4096, m - i), k, device=device) / k ** 0.5).bfloat16()
    for i in range(0, k, 4096):
        b[i:i + 4096] = torch.randn(min(4096, k - i), n, device=device).bfloat16()
    c = gemm(a, b, cfg(256, 256, 64, 4, 2, superblock=1))
    b1 = torch.cat([b[i:i + 4096].sum(dim=1, dtype=torch.float64) for i in range(0, k, 4096)])
    rows = torch.cat([c[i:i + 2048].sum(dim=1, dtype=torch.float64) for i in range(0, m, 2048)])
    want_rows = torch.cat([a[i:i + 2048].double() @ b1 for i in range(0, m, 2048)])
    assert float((rows - want_rows).abs().max() / want_rows.abs().max()) < 4e-3
    a1 = torch.zeros(k, device=device, dtype=torch.float64)
    cols = torch.zeros(n, device=device, dtype=torch.float64)
    for i in range(0, m, 2048):
        a1 += a[i:i + 2048].sum(dim=0, dtype=torch.float64)
        cols += c[i:i + 2048].sum(dim=0, dtype=torch.float64)
    want_cols = torch.zeros(n, device=device, dtype=torch.float64)
    for i in range(0, k, 2048):
        want_cols += a1[i:i + 2048] @ b[i:i + 2048].double()
    assert float((cols - want_cols).abs().max() / want_cols.abs().max()) < 4e-3
    idx = torch.tensor([0, 1, m // 2, m - 2, m - 1], device=device)
    corner = a[idx].float() @ b[:, n - 64:].float()
    assert float((c[idx][:, n - 64:].float() - corner).abs().max() / corner.abs().max()) < 1e-2
    del a, b, c
    torch.cuda.empty_cache()
